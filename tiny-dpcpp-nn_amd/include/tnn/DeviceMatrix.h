// Device memory owners and the non-owning views that are handed to the kernels. Mirrors
// include/common/DeviceMatrix.h of the reference: DeviceMatrixView (:33-59), DeviceMatricesView (:68-109),
// DeviceMatrix (:120-284), DeviceMatrices (:295-499). Memory is hipMalloc'd; element-wise work (fill, the
// packed transposes, type-converting copies) goes through the C ABI of libtnn_hip.
#pragma once

#include <vector>

#include "common.h"

enum class MatrixLayout { RowMajor = 0, ColumnMajor = 1 };

template <typename T> class DeviceMatrixView {
  public:
    DeviceMatrixView() = delete;
    DeviceMatrixView(const size_t m, const size_t n, const size_t stride_col, T *ptr) : m_(m), n_(n), stride_col_(stride_col), ptr_(ptr) {}

    T *GetPointer(const size_t i, const size_t j) const { return ptr_ + j + i * stride_col_; }
    T *GetPointer() const { return ptr_; }

    DeviceMatrixView<T> GetSubMatrix(const size_t m, const size_t n, const size_t offset_m, const size_t offset_n) const {
        return DeviceMatrixView<T>(m, n, stride_col_, ptr_ + offset_n + offset_m * stride_col_);
    }

    size_t m() const { return m_; }
    size_t n() const { return n_; }
    size_t stride() const { return stride_col_; }
    size_t nelements() const { return m() * n(); }

  private:
    size_t m_;
    size_t n_;
    size_t stride_col_;
    T *ptr_;
};

// One input matrix, n_matrices-2 middle matrices and one output matrix in a single allocation.
template <typename T> class DeviceMatricesView {
  public:
    DeviceMatricesView() = delete;
    DeviceMatricesView(const uint32_t n_matrices, const size_t input_m, const size_t input_n, const size_t middle_m,
                       const size_t middle_n, const size_t output_m, const size_t output_n, T *ptr)
        : n_matrices_(n_matrices), input_m_(input_m), input_n_(input_n), middle_m_(middle_m), middle_n_(middle_n),
          output_m_(output_m), output_n_(output_n), ptr_(ptr) {}

    T *GetMatrixPointer(const uint32_t matrix) const {
        if (matrix == 0) return ptr_;
        if (matrix < n_matrices_) return ptr_ + input_m_ * input_n_ + (matrix - 1) * middle_m_ * middle_n_;
        return nullptr;
    }

    T *GetElementPointer(const uint32_t matrix, const size_t row, const size_t col) const {
        T *const mat_ptr = GetMatrixPointer(matrix);
        if (matrix == 0) return mat_ptr + row * input_n_ + col;
        if (matrix == n_matrices_ - 1) return mat_ptr + row * output_n_ + col;
        return mat_ptr + row * middle_n_ + col;
    }

    size_t nelements() const { return input_m_ * input_n_ + output_m_ * output_n_ + (n_matrices_ - 2) * middle_m_ * middle_n_; }
    uint32_t n_matrices() const { return n_matrices_; }
    size_t input_m() const { return input_m_; }
    size_t input_n() const { return input_n_; }
    size_t middle_m() const { return middle_m_; }
    size_t middle_n() const { return middle_n_; }
    size_t output_m() const { return output_m_; }
    size_t output_n() const { return output_n_; }

  private:
    uint32_t n_matrices_;
    size_t input_m_, input_n_, middle_m_, middle_n_, output_m_, output_n_;
    T *ptr_;
};

namespace tnn {
namespace detail {
template <typename T> T *device_alloc(size_t n) {
    void *p = nullptr;
    if (n) hip_check(hipMalloc(&p, n * sizeof(T)), "hipMalloc");
    return static_cast<T *>(p);
}
inline void device_free(void *p) {
    if (p) (void)hipFree(p);
}
} // namespace detail
} // namespace tnn

template <typename T, MatrixLayout _layout = MatrixLayout::RowMajor> class DeviceMatrix {
  public:
    DeviceMatrix(const size_t m, const size_t n, tnn::queue &stream)
        : m_rows(m), m_cols(n), m_q(stream), m_data(tnn::detail::device_alloc<T>(m * n)) {}
    /// A matrix over device memory that somebody else owns (a PyTorch tensor, say) and keeps alive; nothing is freed here.
    DeviceMatrix(const size_t m, const size_t n, tnn::queue &stream, T *borrowed) : m_rows(m), m_cols(n), m_q(stream), m_data(borrowed), m_owns(false) {}
    DeviceMatrix() = delete;
    DeviceMatrix(const DeviceMatrix &other) : m_rows(other.m_rows), m_cols(other.m_cols), m_q(other.m_q), m_data(tnn::detail::device_alloc<T>(other.n_elements())) {
        tnn::hip_check(hipMemcpyAsync(m_data, other.m_data, n_bytes(), hipMemcpyDeviceToDevice, m_q.get()), "hipMemcpyAsync");
        m_q.wait();
    }
    DeviceMatrix(DeviceMatrix &&other) : m_rows(other.m_rows), m_cols(other.m_cols), m_q(other.m_q), m_data(other.m_data), m_owns(other.m_owns) { other.m_data = nullptr; }
    DeviceMatrix &operator=(const DeviceMatrix &other) {
        if (this == &other) return *this;
        if (other.m_rows != m_rows || other.m_cols != m_cols) throw std::invalid_argument("Cannot assign matrices of differing dimensions.");
        tnn::hip_check(hipMemcpyAsync(m_data, other.m_data, n_bytes(), hipMemcpyDeviceToDevice, m_q.get()), "hipMemcpyAsync");
        m_q.wait();
        return *this;
    }
    ~DeviceMatrix() {
        if (m_owns) tnn::detail::device_free(m_data);
    }

    tnn::event fill(const T val) {
        tnn::abi_check(tnn_fill(tnn::dtype_of<T>::value, m_data, n_elements(), (float)val, m_q.abi()));
        return tnn::event(m_q.get());
    }
    // Uniform values in [lower, upper), drawn on the device from a fixed seed (the reference draws from oneMKL philox with
    // seed 777, DeviceMatrix.h:169-178 there; that sequence is not reproducible, the distribution is the same).
    tnn::event fill_random(const T lower_bound, const T upper_bound) {
        tnn::abi_check(tnn_fill_uniform(tnn::dtype_of<T>::value, m_data, n_elements(), (float)lower_bound, (float)upper_bound, 777, 0, m_q.abi()));
        return tnn::event(m_q.get());
    }
    tnn::event copy_to_host(std::vector<T> &out) const {
        if (out.size() < n_elements()) throw std::invalid_argument("Target too small.");
        tnn::hip_check(hipMemcpyAsync(out.data(), m_data, n_bytes(), hipMemcpyDeviceToHost, m_q.get()), "hipMemcpyAsync");
        m_q.wait();
        return tnn::event(m_q.get());
    }
    std::vector<T> copy_to_host() const {
        std::vector<T> v(n_elements());
        copy_to_host(v);
        return v;
    }
    tnn::event copy_from_host(const std::vector<T> &vec) {
        if (vec.size() != n_elements()) throw std::invalid_argument("Vector size does not match matrix size.");
        tnn::hip_check(hipMemcpyAsync(m_data, vec.data(), n_bytes(), hipMemcpyHostToDevice, m_q.get()), "hipMemcpyAsync");
        m_q.wait();
        return tnn::event(m_q.get());
    }
    template <typename Ts> void copy_from_device(Ts const *const src) {
        tnn::abi_check(tnn_cast(tnn::dtype_of<T>::value, m_data, tnn::dtype_of<Ts>::value, src, n_elements(), m_q.abi()));
    }

    T *data() { return m_data; }
    T const *data() const { return m_data; }
    size_t rows() const { return m_rows; }
    size_t m() const { return rows(); }
    size_t cols() const { return m_cols; }
    size_t n() const { return cols(); }
    size_t n_elements() const { return rows() * cols(); }
    size_t size() const { return n_elements(); }
    size_t n_bytes() const { return n_elements() * sizeof(T); }
    constexpr MatrixLayout layout() const { return _layout; }
    tnn::queue &get_queue() { return m_q; }

    DeviceMatrixView<T> GetView() { return GetView(m_rows, m_cols, 0, 0); }
    const DeviceMatrixView<T> GetView() const { return DeviceMatrixView<T>(m_rows, m_cols, m_cols, m_data); }
    DeviceMatricesView<T> GetViews() const { return DeviceMatricesView<T>(1, m(), n(), 0, 0, 0, 0, m_data); }
    DeviceMatrixView<T> GetView(const size_t m, const size_t n, const size_t offset_m, const size_t offset_n) {
        if (offset_m + m > m_rows) throw std::invalid_argument("Potential OOB access.");
        if (offset_n + n > m_cols) throw std::invalid_argument("Potential OOB access.");
        return DeviceMatrixView<T>(m, n, m_cols, m_data + offset_n + offset_m * m_cols);
    }

  private:
    size_t m_rows, m_cols;
    tnn::queue &m_q;
    T *m_data;
    bool m_owns = true;
};

template <typename T> class DeviceMatrices {
  public:
    DeviceMatrices() = delete;
    DeviceMatrices(const uint32_t n_matrices, const size_t input_m, const size_t input_n, const size_t middle_m, const size_t middle_n,
                   const size_t output_m, const size_t output_n, tnn::queue &q)
        : m_q(q), n_matrices_(n_matrices), input_m_(input_m), input_n_(input_n), middle_m_(middle_m), middle_n_(middle_n),
          output_m_(output_m), output_n_(output_n), matrices_(tnn::detail::device_alloc<T>(nelements())) {}
    DeviceMatrices(const DeviceMatrices &) = delete;
    DeviceMatrices(DeviceMatrices &&) = delete;
    DeviceMatrices &operator=(const DeviceMatrices &) = delete;
    DeviceMatrices &operator=(DeviceMatrices &&) = delete;
    ~DeviceMatrices() { tnn::detail::device_free(matrices_); }

    uint32_t GetNumberOfMatrices() const { return n_matrices_; }
    DeviceMatricesView<T> GetViews() const {
        return DeviceMatricesView<T>(n_matrices_, input_m_, input_n_, middle_m_, middle_n_, output_m_, output_n_, matrices_);
    }
    DeviceMatrixView<T> GetView(const uint32_t idx) const {
        if (idx >= n_matrices_) throw std::invalid_argument("Invalid idx");
        if (idx == 0) return DeviceMatrixView<T>(input_m_, input_n_, input_n_, GetMatrixPtr(idx));
        if (idx == n_matrices_ - 1) return DeviceMatrixView<T>(output_m_, output_n_, output_n_, GetMatrixPtr(idx));
        return DeviceMatrixView<T>(middle_m_, middle_n_, middle_n_, GetMatrixPtr(idx));
    }
    DeviceMatrixView<T> Front() const { return GetView(0); }
    DeviceMatrixView<T> Back() const { return GetView(n_matrices_ - 1); }

    // Whole-set layout changes (all matrices must be square and of one size, as they are in a network).
    void PackedTranspose(DeviceMatrices<T> &ret) const { permute(ret, &tnn_packed_transpose); }
    void PackAndTranspose(DeviceMatrices<T> &ret) const {
        if (&ret == this) { // the reference calls it in place (tnn_api.h:599-603); stage through a copy
            DeviceMatrices<T> tmp(n_matrices_, input_m_, input_n_, middle_m_, middle_n_, output_m_, output_n_, m_q);
            tnn::hip_check(hipMemcpyAsync(tmp.matrices_, matrices_, nelements() * sizeof(T), hipMemcpyDeviceToDevice, m_q.get()), "hipMemcpyAsync");
            tmp.permute(ret, &tnn_pack_and_transpose);
            m_q.wait();
            return;
        }
        permute(ret, &tnn_pack_and_transpose);
    }
    void Packed(DeviceMatrices<T> &ret) const { permute(ret, &tnn_pack_weights); }

    tnn::event copy_from_host(const std::vector<T> &src) {
        if (src.size() != nelements()) throw std::invalid_argument("Vector size does not match.");
        tnn::hip_check(hipMemcpyAsync(matrices_, src.data(), nelements() * sizeof(T), hipMemcpyHostToDevice, m_q.get()), "hipMemcpyAsync");
        m_q.wait();
        return tnn::event(m_q.get());
    }
    std::vector<T> copy_to_host() const {
        std::vector<T> v(nelements());
        tnn::hip_check(hipMemcpyAsync(v.data(), matrices_, nelements() * sizeof(T), hipMemcpyDeviceToHost, m_q.get()), "hipMemcpyAsync");
        m_q.wait();
        return v;
    }
    tnn::event fill(const T val) {
        tnn::abi_check(tnn_fill(tnn::dtype_of<T>::value, matrices_, nelements(), (float)val, m_q.abi()));
        return tnn::event(m_q.get());
    }

    size_t nelements() const { return input_m_ * input_n_ + (n_matrices_ - 2) * middle_m_ * middle_n_ + output_m_ * output_n_; }
    size_t input_m() const { return input_m_; }
    size_t input_n() const { return input_n_; }
    size_t middle_m() const { return middle_m_; }
    size_t middle_n() const { return middle_n_; }
    size_t output_m() const { return output_m_; }
    size_t output_n() const { return output_n_; }
    T *data() const { return matrices_; }

    T *GetMatrixPtr(const uint32_t matrix) const {
        if (matrix == 0) return matrices_;
        if (matrix < n_matrices_) return matrices_ + input_m_ * input_n_ + (matrix - 1) * middle_m_ * middle_n_;
        throw std::invalid_argument("matrix does not exist");
    }

  private:
    typedef int (*permute_fn)(int, int, int, const void *, void *, tnn_stream_t);
    void permute(DeviceMatrices<T> &ret, permute_fn fn) const {
        if (ret.n_matrices_ != n_matrices_ || ret.nelements() != nelements()) throw std::invalid_argument("Cannot transpose.");
        const bool square = input_m_ == input_n_ && middle_m_ == middle_n_ && output_m_ == output_n_ &&
                            (n_matrices_ < 3 || middle_m_ == input_m_) && output_m_ == input_m_;
        if (!square) throw std::invalid_argument("Cannot transpose: only sets of equal square matrices are supported.");
        tnn::abi_check(fn(tnn::dtype_of<T>::value, (int)input_m_, (int)n_matrices_, matrices_, ret.matrices_, m_q.abi()));
    }

    tnn::queue &m_q;
    uint32_t n_matrices_;
    size_t input_m_, input_n_, middle_m_, middle_n_, output_m_, output_n_;
    T *matrices_;
};
