// Network base classes of the native C++ API. Mirrors include/network/Network.h of the reference:
// NetworkBase (:20-56) and Network (:59-314) with its width padding, sanity checks, weight initialisation,
// ZeroWeightsPadding and the second, transposed copy of the packed weights. In addition to the two packed
// copies the reference keeps, the network owns the operand-order ("prepared") copies the HIP kernels read;
// they are rebuilt whenever the packed weights change.
#pragma once

#include <random>

#include "DeviceMatrix.h"

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
        : m_q(q), input_width_(CheckedShape(n_hidden_layers, input_width, network_width, output_width)),
          output_width_(PadWidths(output_width, network_width)),
          original_output_width_(output_width), original_input_width_(input_width), n_hidden_layers_(NonNegative(n_hidden_layers)),
          network_width_(NonNegative(network_width)), use_bias_(use_bias),
          m_weights_matrices(get_n_hidden_layers() + 1, get_input_width(), get_network_width(), get_network_width(), get_network_width(),
                             get_network_width(), get_output_width(), m_q),
          m_weightsT_matrices(get_n_hidden_layers() + 1, get_network_width(), get_input_width(), get_network_width(),
                              get_network_width(), get_output_width(), get_network_width(), m_q) {
        SanityCheck();
        tnn::abi_check(tnn_device_check());
        const tnn_mlp_desc d = weights_desc();
        prepared_bytes_ = tnn_mlp_prepared_bytes(&d);
        tnn::hip_check(hipMalloc(&prepared_fwd_, prepared_bytes_), "hipMalloc");
        tnn::hip_check(hipMalloc(&prepared_bwd_, prepared_bytes_), "hipMalloc");
        initialize_weights_matrices(input_width, output_width, mode);
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
            m_weights_matrices.copy_from_host(get_packed_weights<T>(weights, n_hidden_layers_, input_width_, network_width_, output_width_)).wait();
        ZeroWeightsPadding(original_input_width_, original_output_width_);
        TransposeWeights(m_weights_matrices, m_weightsT_matrices);
    }

    /// Same, from parameters that are already on the device (of type T, or fp32 masters that are rounded to T on
    /// the way). No host round trip.
    template <typename Ts> void set_weights_matrices_from_device(Ts const *const d_weights, const bool weights_are_packed) {
        const int dtype = tnn::dtype_of<T>::value;
        const size_t n = m_weights_matrices.nelements();
        if (weights_are_packed) {
            tnn::abi_check(tnn_cast(dtype, m_weights_matrices.data(), tnn::dtype_of<Ts>::value, d_weights, n, m_q.abi()));
        } else { // the transposed copy is rebuilt below; until then it is the staging buffer of the converted values
            tnn::abi_check(tnn_cast(dtype, m_weightsT_matrices.data(), tnn::dtype_of<Ts>::value, d_weights, n, m_q.abi()));
            tnn::abi_check(tnn_pack_weights(dtype, network_width_, n_hidden_layers_ + 1, m_weightsT_matrices.data(), m_weights_matrices.data(), m_q.abi()));
        }
        // everything above and below is enqueued on the one in-order stream: no host wait is needed here
        ZeroWeightsPadding(original_input_width_, original_output_width_, false);
        TransposeWeights(m_weights_matrices, m_weightsT_matrices, false);
    }

    virtual const DeviceMatrices<T> &get_weights_matrices() const { return m_weights_matrices; }
    virtual const DeviceMatrices<T> &get_weightsT_matrices() const { return m_weightsT_matrices; }

    virtual int get_n_hidden_layers() const { return n_hidden_layers_; }
    virtual int get_n_hidden_matrices() const { return n_hidden_layers_ - 1; }
    virtual int get_network_width() const { return network_width_; }
    virtual uint32_t get_input_width() const { return input_width_; }
    virtual uint32_t get_output_width() const { return output_width_; }
    virtual uint32_t get_unpadded_output_width() const { return original_output_width_; }
    virtual uint32_t get_unpadded_input_width() const { return original_input_width_; }

  protected:
    // Operand-order copies of the weights for the forward and the backward kernels.
    const void *prepared_forward() const { return prepared_fwd_; }
    const void *prepared_backward() const { return prepared_bwd_; }

    tnn_mlp_desc weights_desc() const {
        tnn_mlp_desc d;
        d.dtype = tnn::dtype_of<T>::value;
        d.width = network_width_;
        d.n_hidden_layers = n_hidden_layers_;
        d.activation = tnn::to_abi(Activation::None);
        d.output_activation = tnn::to_abi(Activation::None);
        return d;
    }

  private:
    virtual void SanityCheck() const { SanityCheck((int)get_input_width(), (int)get_output_width(), n_hidden_layers_, network_width_); }

    static void SanityCheck(const int input_width, const int output_width, const int n_hidden_layers, const int network_width) {
        if (input_width <= 0)
            throw std::runtime_error("Input width of " + std::to_string(input_width) + " is not supported. Value must be larger than 0.");
        if (output_width <= 0)
            throw std::runtime_error("Output width of " + std::to_string(output_width) + " is not supported. Value must be larger than 0.");
        if (input_width > network_width)
            throw std::runtime_error("Input width of " + std::to_string(input_width) + " is not supported. Value must be <= network width (" +
                                     std::to_string(network_width) + ").");
        if (output_width > network_width)
            throw std::runtime_error("Input width of " + std::to_string(output_width) + " is not supported. Value must be <= network width (" +
                                     std::to_string(network_width) + ").");
        if (n_hidden_layers <= 0)
            throw std::runtime_error("N hidden layers is " + std::to_string(output_width) +
                                     " but must be >= 1, i.e., 1 hidden layer and 1 output layer.");
        if (network_width != 16 && network_width != 32 && network_width != 64 && network_width != 128)
            throw std::invalid_argument("Network width has to be a power of 2 between 16 and 128.");
        if (network_width != input_width || network_width != output_width)
            throw std::invalid_argument("Only networks with same input, layer and output width are allowed.");
    }

    // Runs every check on the shape before the first member allocates device memory (the reference checks after
    // its allocations; the exceptions are the same, in the same order). Returns the padded input width.
    static int CheckedShape(const int n_hidden_layers, const int input_width, const int network_width, const int output_width) {
        const int padded_input = PadWidths(input_width, network_width), padded_output = PadWidths(output_width, network_width);
        NonNegative(n_hidden_layers);
        NonNegative(network_width);
        SanityCheck(padded_input, padded_output, n_hidden_layers, network_width);
        return padded_input;
    }

    /// Zeroes the weights that only see padding: rows of the input matrix at and beyond the one-padded input
    /// width and columns of the output matrix at and beyond the unpadded output width.
    void ZeroWeightsPadding(const int unpadded_input_width, const int unpadded_output_width, const bool wait = true) {
        if (unpadded_input_width > int(get_input_width()) || unpadded_output_width > int(get_output_width()))
            throw std::invalid_argument("Padded weights width cannot be less than the unpadded.");
        constexpr int input_width_divisibly_by = 16;
        int one_padded_input_width = unpadded_input_width;
        if (use_bias_)
            one_padded_input_width = tinydpcppnn::math::next_multiple<int>(unpadded_input_width, input_width_divisibly_by);
        if (one_padded_input_width > int(get_input_width()))
            throw std::invalid_argument("one_padded_input_width > padded_input_width, the input width is too small.");
        const tnn_mlp_desc d = weights_desc();
        tnn::abi_check(tnn_zero_weights_padding(&d, m_weights_matrices.data(), unpadded_input_width, unpadded_output_width, use_bias_ ? 1 : 0, m_q.abi()));
        if (wait) m_q.wait();
    }

    void TransposeWeights(const DeviceMatrices<T> &weights, DeviceMatrices<T> &weightsT, const bool wait = true) {
        weights.PackedTranspose(weightsT);
        const tnn_mlp_desc d = weights_desc();
        tnn::abi_check(tnn_mlp_prepare_weights(&d, weights.data(), 0, prepared_fwd_, prepared_bwd_, m_q.abi()));
        if (wait) m_q.wait();
    }

    void initialize_weights_matrices(const int unpadded_input_width, const int unpadded_output_width, WeightInitMode mode) {
        if (mode == WeightInitMode::arange) {
            throw std::invalid_argument("arange not supported");
        } else if (mode == WeightInitMode::constant_pos) {
            initialize_constant(m_weights_matrices, T(0.01));
        } else if (mode == WeightInitMode::constant_negative) {
            initialize_constant(m_weights_matrices, T(-0.01));
        } else if (mode == WeightInitMode::xavier_normal) {
            initialize_xavier_normal(m_weights_matrices);
        } else if (mode == WeightInitMode::none) {
            initialize_constant(m_weights_matrices, T(1.0));
        } else {
            throw std::invalid_argument("Invalid weights initialization mode.");
        }
        m_q.wait();
        ZeroWeightsPadding(unpadded_input_width, unpadded_output_width);
        TransposeWeights(m_weights_matrices, m_weightsT_matrices);
    }

    static void initialize_constant(DeviceMatrices<T> &ms, const T &constant) { ms.fill(constant); }

    // Uniform in +-sqrt(6 / (fan_in + fan_out)); for the first and the last matrix one fan term is the
    // unpadded input width rounded up to 16 (as in the reference, for both of them).
    void initialize_xavier_normal(DeviceMatrices<T> &ms, const double weight_val_scaling_factor = 1.0) {
        std::random_device rd;
        std::mt19937 gen(rd());
        std::vector<T> weight_matrix_vec(ms.nelements());
        size_t pos = 0;
        for (uint32_t mat_i = 0; mat_i < ms.GetNumberOfMatrices(); ++mat_i) {
            int fan_in_out = network_width_ + network_width_;
            if (mat_i == 0 || mat_i + 1 == ms.GetNumberOfMatrices())
                fan_in_out = tinydpcppnn::math::next_multiple<int>(original_input_width_, 16) + network_width_;
            const double bound = weight_val_scaling_factor * std::sqrt(6.0 / fan_in_out);
            std::uniform_real_distribution<> dis(-bound, bound);
            const size_t n = ms.GetView(mat_i).nelements();
            for (size_t i = 0; i < n; ++i, ++pos) weight_matrix_vec[pos] = static_cast<T>((float)dis(gen));
        }
        ms.copy_from_host(weight_matrix_vec).wait();
    }

    static int PadWidths(const int width, const int base) {
        if (width <= 0) throw std::invalid_argument("width <= 0 cannot be padded.");
        if (base <= 0) throw std::invalid_argument("base <= 0 cannot be used for padding.");
        return ((width + base - 1) / base) * base;
    }

    static int NonNegative(const int number) {
        if (number < 0) throw std::invalid_argument("Use non-negative number.");
        return number;
    }

    tnn::queue &m_q;
    const uint32_t input_width_;
    const uint32_t output_width_;
    const uint32_t original_output_width_;
    const uint32_t original_input_width_;
    const int n_hidden_layers_;
    const int network_width_;
    const bool use_bias_;

    DeviceMatrices<T> m_weights_matrices;
    DeviceMatrices<T> m_weightsT_matrices;
    size_t prepared_bytes_ = 0;
    void *prepared_fwd_ = nullptr;
    void *prepared_bwd_ = nullptr;
};
