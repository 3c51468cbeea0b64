// Device-side building blocks shared by the fused MLP kernels (gfx950): the per-wave 32-row tile in
// MFMA B-operand order, the weight-fragment product, and the activation / rounding steps.
//
// Register layout: lane (j = lane % 32, h = lane / 32) owns batch row j of the wave's tile; for every
// block kb of 16 features it holds the 8 features 16*kb + 8*h + [0, 8): one aligned 16-byte piece of
// the row-major row. Loads, stores and MFMA B operands all use this layout.
#pragma once

#include "tnn_internal.h"

namespace tnn {

constexpr int kFwdThreads = 256;   // streaming kernels: 4 waves per workgroup share one LDS copy of the weights
constexpr int kTrainThreads = 512; // fused training step: 8 waves per workgroup
constexpr int kWaveSize = 64;

// ------------------------------------------------------------------------------------------
// Device helpers
// ------------------------------------------------------------------------------------------

template <int ACT> __device__ __forceinline__ float act_f32(float v) {
    if (ACT == TNN_ACT_RELU) return fmaxf(v, 0.0f);
    if (ACT == TNN_ACT_SIGMOID) return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    return v;
}

typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <typename T> struct Pair;
template <> struct Pair<bf16_t> { typedef bf16x2 type; };
template <> struct Pair<fp16_t> { typedef fp16x2 type; };

// Two fp32 -> one dword holding two values of T (round to nearest even): one packed convert.
template <typename T> __device__ __forceinline__ unsigned int cvt_pair(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, typename Pair<T>::type));
}

// max(v, 0) on two 2-byte floats with one packed 16-bit integer instruction: a negative bf16/fp16 has
// its sign bit set, i.e. is a negative int16, and every non-negative one is a non-negative int16.
__device__ __forceinline__ unsigned int relu_pair(unsigned int v) {
    const s16x2 b = __builtin_elementwise_max(__builtin_bit_cast(s16x2, v), s16x2{0, 0});
    return __builtin_bit_cast(unsigned int, b);
}

// Hides from the optimiser what a value is (here: that a mask is 0 or 1 per half, which it would turn back into
// per-half compares and selects). The statement emits no instruction: the value stays in the register the compiler
// gave it. Instructions written out in inline asm are not an option in these kernels: their destination registers are
// invisible to the compiler's hazard bookkeeping, and one that lands in the unused part of the destination of an MFMA
// still in flight is overwritten when the MFMA retires.
__device__ __forceinline__ unsigned int opaque(unsigned int v) {
    asm("" : "+v"(v));
    return v;
}

// g where fwd > 0, else 0, with packed 16-bit integer instructions: m = min(max(fwd, 0), 1) is 1 exactly
// for the positive values of fwd (as int16), and g * m keeps or clears the bit pattern of g
// (v_pk_max_i16, v_pk_min_i16, v_pk_mul_lo_u16).
__device__ __forceinline__ unsigned int relu_gate_pair(unsigned int g, unsigned int fwd) {
    s16x2 m = __builtin_elementwise_max(__builtin_bit_cast(s16x2, fwd), s16x2{0, 0});
    m = __builtin_elementwise_min(m, __builtin_bit_cast(s16x2, opaque(0x00010001u)));
    const u16x2 r = __builtin_bit_cast(u16x2, g) * __builtin_bit_cast(u16x2, opaque(__builtin_bit_cast(unsigned int, m)));
    return __builtin_bit_cast(unsigned int, r);
}

// The same gate when fwd is known to be the output of relu_pair (never negative, never -0): min(fwd, 1)
// as unsigned 16-bit integers is already the 0/1 mask (v_pk_min_u16, v_pk_mul_lo_u16).
__device__ __forceinline__ unsigned int relu_gate_pair_nonneg(unsigned int g, unsigned int fwd) {
    const u16x2 m = __builtin_elementwise_min(__builtin_bit_cast(u16x2, fwd), __builtin_bit_cast(u16x2, opaque(0x00010001u)));
    const u16x2 r = __builtin_bit_cast(u16x2, g) * __builtin_bit_cast(u16x2, opaque(__builtin_bit_cast(unsigned int, m)));
    return __builtin_bit_cast(unsigned int, r);
}

// Accumulator half (8 fp32 of one 32x32 tile) -> activation -> 8 values of T.
// ReLU before or after the rounding gives the same value (rounding keeps the sign), so it is applied to
// the rounded values, two per instruction.
template <typename T, int ACT, int HALF>
__device__ __forceinline__ typename Storage<T>::vec8 act_convert(const f32x16 &c) {
    u32x4 r;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        float a = c[HALF * 8 + 2 * p], b = c[HALF * 8 + 2 * p + 1];
        if (ACT == TNN_ACT_SIGMOID) {
            a = act_f32<ACT>(a);
            b = act_f32<ACT>(b);
        }
        unsigned int u = cvt_pair<T>(a, b);
        if (ACT == TNN_ACT_RELU) u = relu_pair(u);
        r[p] = u;
    }
    return __builtin_bit_cast(typename Storage<T>::vec8, r);
}

// Backward: fp32 accumulator, masked / scaled by the stored forward activation, then rounded
// (zeroing before or after the rounding is the same). NONNEG: the activation was produced by this
// library's own ReLU in the same kernel.
template <typename T, int ACT, int HALF, bool NONNEG = false>
__device__ __forceinline__ typename Storage<T>::vec8 bwd_convert(const f32x16 &c,
                                                                 const typename Storage<T>::vec8 &fwd) {
    const u32x4 fw = __builtin_bit_cast(u32x4, fwd);
    u32x4 r;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        float a = c[HALF * 8 + 2 * p], b = c[HALF * 8 + 2 * p + 1];
        if (ACT == TNN_ACT_SIGMOID) {
            const float fa = (float)fwd[2 * p], fb = (float)fwd[2 * p + 1];
            a = as_fp32(a * (fa * (1.0f - fa)));
            b = as_fp32(b * (fb * (1.0f - fb)));
        }
        unsigned int u = cvt_pair<T>(a, b);
        if (ACT == TNN_ACT_RELU) u = NONNEG ? relu_gate_pair_nonneg(u, fw[p]) : relu_gate_pair(u, fw[p]);
        r[p] = u;
    }
    return __builtin_bit_cast(typename Storage<T>::vec8, r);
}

// "nt" bit of a buffer store: the line is written through instead of staying dirty in L2 until the kernel ends. Only
// with stores that cover whole 128-byte lines; with partial lines it costs more than it saves.
constexpr int kStreamingStore = 2;

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

    // The same rows through a buffer resource whose range is the matrix (`rows_of`): a lane outside the matrix passes
    // `kNoRow`, its loads return zeros and its stores are dropped by the range check, so the instructions issue
    // unconditionally and the waits on them can count exactly (a load under a branch forces a wait for everything).
    static constexpr unsigned int kNoRow = 0xFFFFFF00u;
    static constexpr unsigned long long kMaxBufferBytes = 1ull << 31;
    static __device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_of(const T *base, long long M) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(base), 0, (int)(unsigned int)(M * W * (long long)sizeof(T)), 0x00020000);
    }
    static __device__ __forceinline__ unsigned int row_offset(long long row, int h, bool valid) {
        return valid ? (unsigned int)(row * (W * (long long)sizeof(T))) + 16u * h : kNoRow;
    }
    template <int AUX = 0>
    static __device__ __forceinline__ void load(vec8 (&r)[NK], __amdgpu_buffer_rsrc_t rows, unsigned int off) {
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) r[kb] = __builtin_bit_cast(vec8, __builtin_amdgcn_raw_buffer_load_b128(rows, off + 32 * kb, 0, AUX));
    }
    template <int AUX = 0>
    static __device__ __forceinline__ void store(const vec8 (&r)[NK], __amdgpu_buffer_rsrc_t rows, unsigned int off) {
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, r[kb]), rows, off + 32 * kb, 0, AUX);
    }

    // Stores of a tile as whole rows: the lane's pieces go to a row-major copy of the tile in LDS (32 rows of PITCH
    // bytes, owned by the wave) and come back with W/8 neighbouring lanes holding one row, so that a store instruction
    // writes complete 128-byte lines instead of 32 bytes of each of 32 lines (measured: 10 % on the backward pass).
    static constexpr int PITCH = W * 2 + 16;  // bytes per staged row (16-byte skew against bank conflicts)
    static constexpr int TILE_BYTES = 32 * PITCH;
    static constexpr int LPR = W / 8;          // lanes per row of 16-byte pieces
    static constexpr int RPI = kWaveSize / LPR; // rows per store instruction; NK instructions per tile
    static __device__ __forceinline__ void row_offsets(unsigned int (&o)[NK], long long tile, int lane, long long M) {
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const long long r = tile * 32 + i * RPI + lane / LPR;
            o[i] = (r < M) ? (unsigned int)(r * (W * (long long)sizeof(T))) + (lane % LPR) * 16 : kNoRow;
        }
    }
    static __device__ __forceinline__ void stage(const vec8 (&r)[NK], unsigned char *tile_lds, int j, int h) {
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) *reinterpret_cast<vec8 *>(tile_lds + j * PITCH + h * 16 + 32 * kb) = r[kb];
    }
    // AUX: cache policy bits of the store; kStreamingStore marks data that this GPU does not read again soon.
    template <int AUX = 0>
    static __device__ __forceinline__ void store_staged(const unsigned char *tile_lds, int lane, __amdgpu_buffer_rsrc_t rows,
                                                        const unsigned int (&o)[NK]) {
#pragma unroll
        for (int i = 0; i < NK; ++i)
            __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(tile_lds + (i * RPI + lane / LPR) * PITCH + (lane % LPR) * 16),
                                                   rows, o[i], 0, AUX);
    }

    // The same store from one offset per tile (that of the lane's 16 bytes in the first of its rows) and a constant per
    // instruction. Rows past the end of the matrix need no flag: their offsets lie past the end of the buffer resource and the
    // range check drops them (the resource covers less than 2^31 bytes, so an offset cannot wrap back into range).
    static __device__ __forceinline__ unsigned int staged_base(long long tile, int lane) {
        return (unsigned int)((tile * 32 + lane / LPR) * (W * (long long)sizeof(T))) + (lane % LPR) * 16;
    }
    template <int AUX = 0>
    static __device__ __forceinline__ void store_staged_at(const unsigned char *tile_lds, int lane, __amdgpu_buffer_rsrc_t rows, unsigned int base) {
#pragma unroll
        for (int i = 0; i < NK; ++i)
            __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4 *>(tile_lds + (i * RPI + lane / LPR) * PITCH + (lane % LPR) * 16),
                                                   rows, base, i * RPI * W * (int)sizeof(T), AUX);
    }

    static constexpr int NF = NI * NK; // weight fragments per matrix and lane

    // The lane's NF operand fragments of matrix l (LDS or global, already in operand order).
    static __device__ __forceinline__ void load_frags(vec8 (&f)[NF], const vec8 *__restrict__ w, int l, int lane) {
        const vec8 *p = w + (size_t)l * (NF * kWaveSize) + lane;
#pragma unroll
        for (int i = 0; i < NF; ++i) f[i] = p[i * kWaveSize];
    }

    // acc[a] = sum_kb frag(a, kb) * b[kb]
    static __device__ __forceinline__ void mma(f32x16 (&acc)[NI], const vec8 (&b)[NK], const vec8 (&f)[NF]) {
#pragma unroll
        for (int a = 0; a < NI; ++a) acc[a] = f32x16{};
#pragma unroll
        for (int kb = 0; kb < NK; ++kb) {
#pragma unroll
            for (int a = 0; a < NI; ++a) acc[a] = Storage<T>::mfma(f[a * NK + kb], b[kb], acc[a]);
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

    template <int ACT, bool NONNEG = false>
    static __device__ __forceinline__ void bwd_repack(vec8 (&r)[NK], const f32x16 (&acc)[NI], const vec8 (&fwd)[NK]) {
#pragma unroll
        for (int a = 0; a < NI; ++a) {
            r[2 * a] = bwd_convert<T, ACT, 0, NONNEG>(acc[a], fwd[2 * a]);
            if (2 * a + 1 < NK) r[2 * a + 1] = bwd_convert<T, ACT, 1, NONNEG>(acc[a], fwd[2 * a + 1 < NK ? 2 * a + 1 : 0]);
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
