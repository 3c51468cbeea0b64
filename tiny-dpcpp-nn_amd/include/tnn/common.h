// Host-side common definitions of the native C++ API (namespace-free where the reference is, so that
// code written against the reference's headers reads the same). Mirrors include/common/common.h of the
// reference: the Activation enum (:28-38), the math helpers (:49-75), the packed-layout coordinate maps
// (source/common/common.cpp:33-66) and get_packed_weights (:174-212). The SYCL queue of the reference
// becomes tnn::queue, a thin handle around a hipStream_t.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "tnn_hip.h"

enum class Activation {
    ReLU,
    LeakyReLU,
    Exponential,
    Sine,
    Sigmoid,
    Squareplus,
    Softplus,
    Tanh,
    None,
};

// Base of the per-call contexts handed around by encodings (reference: common.h:40-47).
struct Context {
    Context() = default;
    virtual ~Context() {}
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
};

namespace tnn {

// 16-bit storage types on the host. Conversions round to nearest even, like the device.
struct bf16 {
    uint16_t bits = 0;
    bf16() = default;
    bf16(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        if ((u & 0x7f800000u) == 0x7f800000u) {
            bits = (uint16_t)((u >> 16) | ((u & 0x007fffffu) ? 0x40 : 0));
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            bits = (uint16_t)(u >> 16);
        }
    }
    bf16(double d) : bf16((float)d) {}
    bf16(int i) : bf16((float)i) {}
    operator float() const {
        const uint32_t u = (uint32_t)bits << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

struct half {
    uint16_t bits = 0;
    half() = default;
    half(float f) {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        const uint32_t sign = (u >> 16) & 0x8000u;
        uint32_t a = u & 0x7fffffffu;
        if (a >= 0x7f800000u) {
            bits = (uint16_t)(sign | 0x7c00u | ((a > 0x7f800000u) ? 0x200u : 0));
        } else if (a >= 0x477ff000u) {
            bits = (uint16_t)(sign | 0x7c00u);
        } else if (a >= 0x38800000u) {
            a += 0xfffu + ((a >> 13) & 1u);
            bits = (uint16_t)(sign | ((a - 0x38000000u) >> 13));
        } else {
            float av;
            std::memcpy(&av, &a, 4);
            volatile float t = av + 0.5f; // quantum of [0.5, 1) is 2^-24, the half denormal step
            const float r = t - 0.5f;
            bits = (uint16_t)(sign | (uint16_t)std::lrintf(r * 16777216.0f));
        }
    }
    half(double d) : half((float)d) {}
    half(int i) : half((float)i) {}
    operator float() const {
        const uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
        const uint32_t e = (bits >> 10) & 0x1f, m = bits & 0x3ffu;
        float f;
        if (e == 0) {
            f = std::ldexp((float)m, -24);
        } else if (e == 31) {
            const uint32_t u = 0x7f800000u | (m << 13);
            std::memcpy(&f, &u, 4);
        } else {
            const uint32_t u = ((e + 112) << 23) | (m << 13);
            std::memcpy(&f, &u, 4);
        }
        uint32_t u;
        std::memcpy(&u, &f, 4);
        u |= sign;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

template <typename T> struct dtype_of;
template <> struct dtype_of<bf16> { static constexpr int value = TNN_BF16; };
template <> struct dtype_of<half> { static constexpr int value = TNN_FP16; };
template <> struct dtype_of<float> { static constexpr int value = TNN_FP32; };

// Stands where the reference passes a sycl::queue&: a non-owning handle of the stream all work goes to.
class queue {
  public:
    queue() = default;
    explicit queue(hipStream_t s) : stream_(s) {}
    hipStream_t get() const { return stream_; }
    void rebind(hipStream_t s) { stream_ = s; } // every holder of a reference to this queue follows
    tnn_stream_t abi() const { return reinterpret_cast<tnn_stream_t>(stream_); }
    void wait() const {
        if (hipStreamSynchronize(stream_) != hipSuccess) throw std::runtime_error("hipStreamSynchronize failed");
    }

  private:
    hipStream_t stream_ = nullptr;
};

// Stands where the reference returns a sycl::event: waiting on it waits for the work enqueued so far.
class event {
  public:
    event() = default;
    explicit event(hipStream_t s) : stream_(s) {}
    void wait() const {
        if (hipStreamSynchronize(stream_) != hipSuccess) throw std::runtime_error("hipStreamSynchronize failed");
    }

  private:
    hipStream_t stream_ = nullptr;
};

inline void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// Turns a C-ABI status into the exception type the reference throws at the same place.
inline void abi_check(int status) {
    if (status >= 0) return;
    const std::string msg = tnn_last_error();
    if (status == TNN_ERR_INVALID_ARGUMENT || status == TNN_ERR_UNSUPPORTED) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

inline int to_abi(Activation a) { return static_cast<int>(a); }

} // namespace tnn

/// some common math functions (reference: common.h:49-75)
namespace tinydpcppnn {
namespace math {
template <typename T> T div_round_up(T val, T divisor) { return (val + divisor - 1) / divisor; }
template <typename T> T next_multiple(T val, T divisor) { return div_round_up(val, divisor) * divisor; }
template <typename T> T previous_multiple(T val, T divisor) { return (val / divisor) * divisor; }
inline uint32_t powi(uint32_t base, uint32_t exponent) {
    uint32_t result = 1;
    for (uint32_t i = 0; i < exponent; ++i) result *= base;
    return result;
}
} // namespace math
} // namespace tinydpcppnn

// source/common/common.cpp:33-42
inline unsigned toPackedLayoutCoord(const unsigned idx, const unsigned rows, const unsigned cols) {
    (void)rows;
    const unsigned i = idx / cols, j = idx % cols;
    return (i % 2 == 0) ? i * cols + 2 * j : (i - 1) * cols + 2 * j + 1;
}

// source/common/common.cpp:58-66
inline unsigned fromPackedLayoutCoord(const unsigned idx, const unsigned rows, const unsigned cols) {
    (void)rows;
    const unsigned i = idx / (cols * 2), j = idx % (cols * 2);
    return (j % 2 == 0) ? (i * 2) * cols + j / 2 : (i * 2 + 1) * cols + (j - 1) / 2;
}

// common.h:174-182
template <typename T> std::vector<T> vertical_pack(const std::vector<T> &matrix, int rows, int cols) {
    std::vector<T> packed(rows * cols, T(0.0f));
    for (int idx = 0; idx < rows * cols; ++idx) packed[toPackedLayoutCoord(idx, rows, cols)] = matrix[idx];
    return packed;
}

// common.h:184-212: unpacked [in][out] matrices (input, hidden..., output) -> packed parameter vector
template <typename T>
std::vector<T> get_packed_weights(const std::vector<T> &unpacked_weights, int m_n_hidden_layers, int input_width, int network_width,
                                  int output_width) {
    std::vector<T> weights_packed;
    const size_t expected = (size_t)input_width * network_width + (size_t)(m_n_hidden_layers - 1) * network_width * network_width +
                            (size_t)network_width * output_width;
    if (unpacked_weights.size() != expected) throw std::invalid_argument("get_packed_weights: size mismatch");
    std::vector<T> input_matrix(unpacked_weights.begin(), unpacked_weights.begin() + (size_t)input_width * network_width);
    weights_packed = vertical_pack(input_matrix, network_width, input_width);
    const size_t len_input = input_matrix.size();
    for (int layer = 0; layer < m_n_hidden_layers - 1; ++layer) {
        const size_t start = len_input + (size_t)layer * network_width * network_width;
        std::vector<T> hidden(unpacked_weights.begin() + start, unpacked_weights.begin() + start + (size_t)network_width * network_width);
        const std::vector<T> packed_hidden = vertical_pack(hidden, network_width, network_width);
        weights_packed.insert(weights_packed.end(), packed_hidden.begin(), packed_hidden.end());
    }
    std::vector<T> output_matrix(unpacked_weights.end() - (size_t)network_width * output_width, unpacked_weights.end());
    const std::vector<T> packed_output = vertical_pack(output_matrix, network_width, output_width);
    weights_packed.insert(weights_packed.end(), packed_output.begin(), packed_output.end());
    return weights_packed;
}

inline bool isequalstring(const std::string &a, const std::string &b) {
    if (a.size() != b.size()) return false;
    for (size_t i = 0; i < a.size(); ++i)
        if (std::tolower((unsigned char)a[i]) != std::tolower((unsigned char)b[i])) return false;
    return true;
}
