// Network base classes of the native C++ API. The public surface is that of include/network/Network.h of the reference
// (NetworkBase :20-56, Network :59-127): same methods, same widths and paddings, the packed weights and their
// transposed copy. Behind it, everything happens on the device: the shape is checked once before anything is
// allocated, the initial weights are drawn by a seeded kernel, and besides the two packed copies the network owns the
// operand-order ("prepared") copies the HIP kernels read, rebuilt whenever the packed weights change.
#pragma once

#include <atomic>
#include <cstdint>
#include <random>
#include <string>

#include "DeviceMatrix.h"

namespace tnn {
/// Where the seeds of the initial weights come from: std::random_device, as the reference's (Network.h:262-263 there), until
/// set_initial_weight_seed() is called; from then on every network takes the next value of a counter that starts at the given
/// seed, so that a program (a test, a run that is to be repeated) gets the same networks every time.
struct InitialWeightSeed {
    static std::atomic<bool> &fixed() {
        static std::atomic<bool> f{false};
        return f;
    }
    static std::atomic<uint64_t> &counter() {
        static std::atomic<uint64_t> c{0};
        return c;
    }
    static uint64_t next() {
        if (fixed().load()) return counter().fetch_add(1);
        std::random_device entropy;
        return ((uint64_t)entropy() << 32) | (uint64_t)entropy();
    }
};
inline void set_initial_weight_seed(const uint64_t seed) {
    InitialWeightSeed::counter().store(seed);
    InitialWeightSeed::fixed().store(true);
}
} // namespace tnn

template <typename T> class NetworkBase {
  public:
    NetworkBase() {}
    virtual ~NetworkBase() {}

    virtual std::vector<tnn::event> forward_pass(const DeviceMatrix<T> &input, DeviceMatrices<T> &intermediate_output_forward,
                                                 const std::vector<tnn::event> &deps) = 0;
    virtual std::vector<tnn::event> forward_pass(const DeviceMatrixView<T> &input, DeviceMatricesView<T> intermediate_output_forward,
                                                 const std::vector<tnn::event> &deps) = 0;
    virtual std::vector<tnn::event> inference(const DeviceMatrix<T> &input, DeviceMatrix<T> &output,
                                              const std::vector<tnn::event> &deps) = 0;
    virtual std::vector<tnn::event> inference(const DeviceMatrixView<T> &input, DeviceMatricesView<T> output,
                                              const std::vector<tnn::event> &deps) = 0;
    /// input: derivatives of the loss w.r.t. the network output. output: the weight gradients,
    /// per matrix [out][in] row-major, unpacked.
    virtual std::vector<tnn::event> backward_pass(const DeviceMatrix<T> &input, DeviceMatrices<T> &output,
                                                  DeviceMatrices<T> &intermediate_output_backward,
                                                  const DeviceMatrices<T> &intermediate_output_forward,
                                                  const std::vector<tnn::event> &deps, DeviceMatrixView<T> *dL_dinput = nullptr) = 0;
    virtual std::vector<tnn::event> backward_pass(const DeviceMatrixView<T> input, DeviceMatricesView<T> output,
                                                  DeviceMatricesView<T> intermediate_output_backward,
                                                  const DeviceMatricesView<T> intermediate_output_forward,
                                                  const std::vector<tnn::event> &deps, DeviceMatrixView<T> *dL_dinput = nullptr) = 0;
};

template <typename T> class Network : public NetworkBase<T> {
  public:
    enum WeightInitMode { arange, constant_pos, constant_negative, xavier_normal, none };

    Network(tnn::queue &q, const int n_hidden_layers, const int input_width, const int network_width, const int output_width,
            const WeightInitMode mode, const bool use_bias)
        : m_q(q), shape_(Shape::checked(n_hidden_layers, input_width, network_width, output_width, use_bias)),
          m_weights_matrices(shape_.hidden + 1, shape_.in, shape_.width, shape_.width, shape_.width, shape_.width, shape_.out, m_q),
          m_weightsT_matrices(shape_.hidden + 1, shape_.width, shape_.in, shape_.width, shape_.width, shape_.out, shape_.width, m_q) {
        tnn::abi_check(tnn_device_check());
        const tnn_mlp_desc d = weights_desc();
        prepared_bytes_ = tnn_mlp_prepared_bytes(&d);
        tnn::hip_check(hipMalloc(&prepared_fwd_, prepared_bytes_), "hipMalloc");
        tnn::hip_check(hipMalloc(&prepared_bwd_, prepared_bytes_), "hipMalloc");
        draw_initial_weights(mode);
        finish_weights(/*wait=*/true);
    }
    Network(const Network &) = delete;
    Network &operator=(const Network &) = delete;

    virtual ~Network() {
        tnn::detail::device_free(prepared_fwd_);
        tnn::detail::device_free(prepared_bwd_);
    }

    tnn::queue &get_queue() { return m_q; }
    const tnn::queue &get_queue() const { return m_q; }

    /// weights_are_packed == false: `weights` is the flat list of [in][out] matrices (input, hidden..., output).
    virtual void set_weights_matrices(const std::vector<T> &weights, const bool weights_are_packed) {
        if (m_weights_matrices.nelements() != weights.size()) {
            throw std::runtime_error("m_weights_matrices nelements: " + std::to_string(m_weights_matrices.nelements()) +
                                     " does not match unpacked_weights size: " + std::to_string(weights.size()) +
                                     ". Consider padding input and output to have the same amount as network_width");
        }
        if (weights_are_packed)
            m_weights_matrices.copy_from_host(weights).wait();
        else
            m_weights_matrices.copy_from_host(get_packed_weights<T>(weights, shape_.hidden, shape_.in, shape_.width, shape_.out)).wait();
        finish_weights(/*wait=*/true);
    }

    /// Same, from parameters that are already on the device (of type T, or fp32 masters that are rounded to T on
    /// the way). No host round trip.
    template <typename Ts> void set_weights_matrices_from_device(Ts const *const d_weights, const bool weights_are_packed) {
        const int dtype = tnn::dtype_of<T>::value;
        const size_t n = m_weights_matrices.nelements();
        if (weights_are_packed) { // the route of every forward pass of a Python module: one launch for all four copies
            const tnn_mlp_desc d = weights_desc();
            tnn::abi_check(tnn_mlp_set_packed_weights(&d, d_weights, tnn::dtype_of<Ts>::value, (int)shape_.raw_in, (int)shape_.raw_out, shape_.bias ? 1 : 0,
                                                      m_weights_matrices.data(), m_weightsT_matrices.data(), prepared_fwd_, prepared_bwd_, m_q.abi()));
            return;
        } else { // the transposed copy is rebuilt below; until then it is the staging buffer of the converted values
            tnn::abi_check(tnn_cast(dtype, m_weightsT_matrices.data(), tnn::dtype_of<Ts>::value, d_weights, n, m_q.abi()));
            tnn::abi_check(tnn_pack_weights(dtype, shape_.width, shape_.hidden + 1, m_weightsT_matrices.data(), m_weights_matrices.data(), m_q.abi()));
        }
        // everything above and below is enqueued on the one in-order stream: no host wait is needed here
        finish_weights(/*wait=*/false);
    }

    virtual const DeviceMatrices<T> &get_weights_matrices() const { return m_weights_matrices; }
    virtual const DeviceMatrices<T> &get_weightsT_matrices() const { return m_weightsT_matrices; }

    virtual int get_n_hidden_layers() const { return shape_.hidden; }
    virtual int get_n_hidden_matrices() const { return shape_.hidden - 1; }
    virtual int get_network_width() const { return shape_.width; }
    virtual uint32_t get_input_width() const { return shape_.in; }
    virtual uint32_t get_output_width() const { return shape_.out; }
    virtual uint32_t get_unpadded_output_width() const { return shape_.raw_out; }
    virtual uint32_t get_unpadded_input_width() const { return shape_.raw_in; }

  protected:
    // Operand-order copies of the weights for the forward and the backward kernels.
    const void *prepared_forward() const { return prepared_fwd_; }
    const void *prepared_backward() const { return prepared_bwd_; }

    tnn_mlp_desc weights_desc() const {
        tnn_mlp_desc d;
        d.dtype = tnn::dtype_of<T>::value;
        d.width = shape_.width;
        d.n_hidden_layers = shape_.hidden;
        d.activation = tnn::to_abi(Activation::None);
        d.output_activation = tnn::to_abi(Activation::None);
        return d;
    }

  private:
    /// What a derived network adds to the shape checks (its activations, say); the shape itself is checked by Shape::checked.
    virtual void SanityCheck() const {}

    // Everything about the network that is fixed at construction, checked before the first device allocation.
    // Exception types follow the reference's constructor chain (Network.h:59-88,129-167 there): std::invalid_argument for
    // arguments that cannot be padded or counted, std::runtime_error for a shape the kernels do not have.
    struct Shape {
        int hidden = 0, width = 0;
        uint32_t in = 0, out = 0;         // as the kernels see them: padded to the network width
        uint32_t raw_in = 0, raw_out = 0; // as the caller gave them
        bool bias = false;

        static uint32_t round_up(const int value, const int multiple_of, const char *what) {
            if (value <= 0) throw std::invalid_argument(std::string(what) + " width <= 0 cannot be padded.");
            return (uint32_t)((value + multiple_of - 1) / multiple_of * multiple_of);
        }

        static Shape checked(const int n_hidden_layers, const int input_width, const int network_width, const int output_width, const bool use_bias) {
            if (network_width < 0 || n_hidden_layers < 0) throw std::invalid_argument("Use non-negative number for the network width and the layer count.");
            if (network_width != 16 && network_width != 32 && network_width != 64 && network_width != 128)
                throw std::invalid_argument("Network width has to be a power of 2 between 16 and 128, got " + std::to_string(network_width) + ".");
            Shape s;
            s.hidden = n_hidden_layers;
            s.width = network_width;
            s.raw_in = (uint32_t)input_width;
            s.raw_out = (uint32_t)output_width;
            s.in = round_up(input_width, network_width, "Input");
            s.out = round_up(output_width, network_width, "Output");
            if ((int)s.in != network_width)
                throw std::runtime_error("Input width of " + std::to_string(s.in) + " (padded from " + std::to_string(input_width) +
                                         ") is not supported: it must not exceed the network width " + std::to_string(network_width) + ".");
            if ((int)s.out != network_width)
                throw std::runtime_error("Output width of " + std::to_string(s.out) + " (padded from " + std::to_string(output_width) +
                                         ") is not supported: it must not exceed the network width " + std::to_string(network_width) + ".");
            if (n_hidden_layers < 1)
                throw std::runtime_error("N hidden layers is " + std::to_string(n_hidden_layers) + " but must be >= 1, i.e., 1 hidden layer and 1 output layer.");
            s.bias = use_bias;
            return s;
        }
    };

    /// After the packed weights changed: zero what only sees padding (rows of the first matrix that only see padding, columns of
    /// the last matrix from the caller's output width on; Network.h:171-233 of the reference), then rebuild the transposed
    /// packed copy and the two operand-order copies the kernels read. All on the network's stream.
    void finish_weights(const bool wait) {
        const tnn_mlp_desc d = weights_desc();
        tnn::abi_check(tnn_zero_weights_padding(&d, m_weights_matrices.data(), (int)shape_.raw_in, (int)shape_.raw_out, shape_.bias ? 1 : 0, m_q.abi()));
        m_weights_matrices.PackedTranspose(m_weightsT_matrices);
        tnn::abi_check(tnn_mlp_prepare_weights(&d, m_weights_matrices.data(), 0, prepared_fwd_, prepared_bwd_, m_q.abi()));
        if (wait) m_q.wait();
    }

    /// The initial packed weights, drawn on the device. xavier_normal (the reference's name for it) is uniform in
    /// +-sqrt(6 / (fan_in + fan_out)), where the first and the last matrix both count the caller's input width rounded up to
    /// 16 as one of the two fans (Network.h:278-286 there). The seed comes from std::random_device, as the reference's does, unless
    /// tnn::set_initial_weight_seed() fixed it.
    void draw_initial_weights(const WeightInitMode mode) {
        const int dtype = tnn::dtype_of<T>::value;
        switch (mode) {
        case WeightInitMode::constant_pos: m_weights_matrices.fill(T(0.01f)); return;
        case WeightInitMode::constant_negative: m_weights_matrices.fill(T(-0.01f)); return;
        case WeightInitMode::none: m_weights_matrices.fill(T(1.0f)); return;
        case WeightInitMode::arange: throw std::invalid_argument("arange not supported");
        case WeightInitMode::xavier_normal: break;
        default: throw std::invalid_argument("Invalid weights initialization mode.");
        }
        const uint64_t seed = tnn::InitialWeightSeed::next();
        const uint32_t n_mats = m_weights_matrices.GetNumberOfMatrices();
        const int edge_fan = (int)Shape::round_up((int)shape_.raw_in, 16, "Input");
        uint64_t drawn = 0;
        for (uint32_t m = 0; m < n_mats; ++m) {
            const auto view = m_weights_matrices.GetView(m);
            const bool edge = (m == 0 || m + 1 == n_mats);
            const float bound = (float)std::sqrt(6.0 / (double)((edge ? edge_fan : shape_.width) + shape_.width));
            tnn::abi_check(tnn_fill_uniform(dtype, view.GetPointer(), view.nelements(), -bound, bound, seed, drawn, m_q.abi()));
            drawn += view.nelements();
        }
    }

    tnn::queue &m_q;
    const Shape shape_;

    DeviceMatrices<T> m_weights_matrices;
    DeviceMatrices<T> m_weightsT_matrices;
    size_t prepared_bytes_ = 0;
    void *prepared_fwd_ = nullptr;
    void *prepared_bwd_ = nullptr;
};
