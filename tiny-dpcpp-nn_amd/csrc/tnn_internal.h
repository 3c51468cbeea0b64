// Internal helpers shared by the HIP translation units of libtnn_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "tnn_hip.h"

#define TNN_API extern "C" __attribute__((visibility("default")))

namespace tnn {

// Thread-local error text behind tnn_last_error().
char *error_buffer();
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

inline hipStream_t as_stream(tnn_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Reports a failed launch as TNN_ERR_HIP. Does not synchronize.
int check_launch(const char *what);

// Every kernel goes out through this: an error that an earlier, unrelated runtime call of this thread left
// behind (a failed allocation of the caller, say) is dropped first, so that check_launch reports this launch only.
#define TNN_LAUNCH(...)                                                                                                \
    do {                                                                                                               \
        (void)hipGetLastError();                                                                                       \
        hipLaunchKernelGGL(__VA_ARGS__);                                                                               \
    } while (0)

inline bool valid_width(int w) { return w == 16 || w == 32 || w == 64 || w == 128; }
inline bool valid_act(int a) { return a == TNN_ACT_NONE || a == TNN_ACT_RELU || a == TNN_ACT_SIGMOID; }
int check_mlp_desc(const tnn_mlp_desc *d);

typedef __bf16 bf16_t;
typedef _Float16 fp16_t;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 fp16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 fp16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 fp16x2 __attribute__((ext_vector_type(2)));

// Per storage type: 8-wide vector, the 32x32x16 MFMA and the 16x16x32 MFMA (fp32 accumulate).
template <typename T> struct Storage;
template <> struct Storage<bf16_t> {
    typedef bf16x8 vec8;
    typedef bf16x4 vec4;
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Storage<fp16_t> {
    typedef fp16x8 vec8;
    typedef fp16x4 vec4;
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

// Pins a value in a VGPR as an fp32 number. The reference rounds an fp32 product to fp32 first and to the
// 2-byte type afterwards; without this the compiler merges "multiply, then narrow" into one mixed-precision
// instruction that rounds once, which differs on exact ties.
__device__ __forceinline__ float as_fp32(float v) {
    asm volatile("" : "+v"(v));
    return v;
}

// Swaps bits 2 and 3 of a 5-bit index. Row i of a 32-row MFMA output tile is held by lane half
// h = bit 2 in accumulator register 4*(i>>3) + (i&3); storing weight column (32a + swap23(i)) in
// operand row i makes every lane end up with 8 consecutive features per 16-feature block, which is
// exactly the operand order of the next layer and the row-major order in memory.
__host__ __device__ inline int swap23(int i) { return (i & 0x13) | ((i & 4) << 1) | ((i & 8) >> 1); }

// Packed ("VNNI") coordinate of element (k, n) of a W x W matrix.
__host__ __device__ inline int packed_coord(int k, int n, int W) { return (k & ~1) * W + 2 * n + (k & 1); }

} // namespace tnn
