// The fully fused MLP of the native C++ API. Mirrors include/network/SwiftNetMLP.h of the reference
// (constructor :50-58, forward_pass :69-119, inference :135-186, backward_pass :199-257, sanity checks
// :259-418, create_network :424-429). Where the reference instantiates one ESIMD kernel per activation
// pair, this class fills a descriptor and calls the HIP kernels through the C ABI of libtnn_hip.
#pragma once

#include <cstring>

#include <memory>

#include "Network.h"

template <typename T, int WIDTH> class SwiftNetMLP : public Network<T> {
  public:
    SwiftNetMLP(tnn::queue &q, const int input_width, const int output_width, const int n_hidden_layers, Activation activation,
                Activation output_activation, const typename Network<T>::WeightInitMode mode = Network<T>::WeightInitMode::xavier_normal,
                const bool use_bias = false)
        : Network<T>(q, n_hidden_layers, input_width, WIDTH, output_width, mode, use_bias), m_activation{activation},
          m_output_activation{output_activation} {
        SanityCheck();
    }

    ~SwiftNetMLP() { tnn::detail::device_free(workspace_); }

    /// Forward pass that keeps the input and every activated layer output in `intermediate_output_forward`;
    /// the network output is its last matrix.
    std::vector<tnn::event> forward_pass(const DeviceMatrix<T> &input, DeviceMatrices<T> &intermediate_output_forward,
                                         const std::vector<tnn::event> &deps) override {
        SanityCheckForward(input, intermediate_output_forward);
        return forward_pass(input.GetView(), intermediate_output_forward.GetViews(), deps);
    }

    std::vector<tnn::event> forward_pass(const DeviceMatrixView<T> &input, DeviceMatricesView<T> intermediate_output_forward,
                                         const std::vector<tnn::event> &) override {
        RequireDense(input);
        const tnn_mlp_desc d = desc();
        tnn::abi_check(tnn_mlp_forward(&d, this->prepared_forward(), input.GetPointer(), intermediate_output_forward.GetMatrixPointer(0),
                                       input.m(), this->get_queue().abi()));
        return {tnn::event(this->get_queue().get())};
    }

    /// Inference: only the network output is written (to matrix 0 of the output view).
    std::vector<tnn::event> inference(const DeviceMatrix<T> &input, DeviceMatrix<T> &output, const std::vector<tnn::event> &deps) override {
        SanityCheckInference(input, output);
        return inference(input.GetView(), output.GetViews(), deps);
    }

    std::vector<tnn::event> inference(const DeviceMatrixView<T> &input, DeviceMatricesView<T> output,
                                      const std::vector<tnn::event> &) override {
        RequireDense(input);
        const tnn_mlp_desc d = desc();
        tnn::abi_check(tnn_mlp_inference(&d, this->prepared_forward(), input.GetPointer(), output.GetMatrixPointer(0), input.m(),
                                         this->get_queue().abi()));
        return {tnn::event(this->get_queue().get())};
    }

    /// Whether inference_with_grid runs for this grid (its features fit the input width, the weights fit LDS).
    bool supports_grid_input(const tnn_grid_desc &grid) const {
        const tnn_mlp_desc d = desc();
        return Network<T>::get_input_width() == WIDTH && tnn_grid_mlp_supported(&grid, &d) == TNN_OK;
    }

    /// Inference on the grid encoding of `positions` (M x n_dims fp32) without the encoded matrix ever being stored:
    /// the same values as the encoding's forward_impl into a WIDTH-wide matrix of T followed by inference().
    /// No counterpart in the reference, which runs the two kernels (dpcpp_bindings/tiny_dpcpp_nn/modules.py:357-421).
    /// Batches from 2^18 rows on are visited in cell order (ordering 25 us + 45 us against 89 us at 2^18 points of a 2-D grid of
    /// 16 levels); with `a_backward_pass_follows` from 2^17 on, the size from which backward_with_grid orders the batch anyway
    /// and can take this call's order over.
    std::vector<tnn::event> inference_with_grid(const tnn_grid_desc &grid, const void *table, const float *positions, const size_t M,
                                                DeviceMatricesView<T> output, const bool a_backward_pass_follows = false) {
        if (Network<T>::get_input_width() != WIDTH) throw std::invalid_argument("The encoding must be padded to the network width.");
        const tnn_mlp_desc d = desc();
        if (M >= (size_t(1) << (a_backward_pass_follows ? 17 : 18))) {
            // large batches: points in cell order gather from shared lines of the table (same rows, bit for bit)
            OrderPoints(grid, positions, M);
            tnn::abi_check(tnn_grid_mlp_inference_ordered(&grid, &d, m_grid_order->data(), table, this->prepared_forward(),
                                                          output.GetMatrixPointer(0), M, this->get_queue().abi()));
        } else {
            tnn::abi_check(tnn_grid_mlp_inference(&grid, &d, positions, table, this->prepared_forward(), output.GetMatrixPointer(0), M,
                                                  this->get_queue().abi()));
        }
        return {tnn::event(this->get_queue().get())};
    }

    /// input: dL/d(output). output: weight gradients, per matrix [out][in] row-major, unpacked.
    std::vector<tnn::event> backward_pass(const DeviceMatrix<T> &input, DeviceMatrices<T> &output,
                                          DeviceMatrices<T> &intermediate_output_backward,
                                          const DeviceMatrices<T> &intermediate_output_forward, const std::vector<tnn::event> &deps,
                                          DeviceMatrixView<T> *dL_dinput = nullptr) override {
        SanityCheckBackward(input, output, intermediate_output_backward, intermediate_output_forward);
        return backward_pass(input.GetView(), output.GetViews(), intermediate_output_backward.GetViews(),
                             intermediate_output_forward.GetViews(), deps, dL_dinput);
    }

    std::vector<tnn::event> backward_pass(const DeviceMatrixView<T> input, DeviceMatricesView<T> output,
                                          DeviceMatricesView<T> intermediate_output_backward,
                                          const DeviceMatricesView<T> intermediate_output_forward, const std::vector<tnn::event> &,
                                          DeviceMatrixView<T> *dL_dinput = nullptr) override {
        RequireDense(input);
        if (dL_dinput != nullptr) RequireDense(*dL_dinput);
        const tnn_mlp_desc d = desc();
        ReserveWorkspace(tnn_mlp_backward_workspace_bytes(&d, input.m()));
        tnn::abi_check(tnn_mlp_backward(&d, this->prepared_backward(), input.GetPointer(), intermediate_output_forward.GetMatrixPointer(0),
                                        intermediate_output_backward.GetMatrixPointer(0), output.GetMatrixPointer(0), 0,
                                        dL_dinput ? dL_dinput->GetPointer() : nullptr, input.m(), workspace_, workspace_bytes_,
                                        this->get_queue().abi()));
        return {tnn::event(this->get_queue().get())};
    }

    /// Whether backward_pass_recompute runs for this network (the shapes of the one-kernel training step).
    bool supports_backward_recompute() const {
        const tnn_mlp_desc d = desc();
        return Network<T>::get_input_width() == WIDTH && tnn_mlp_backward_recompute_supported(&d) == TNN_OK;
    }

    /// backward_pass for a caller that kept no activations: weight gradients (raw layout, as backward_pass writes them) and,
    /// on request, dL/dinput for `dL_doutput`, the activations being formed again on chip from `input` (the matrix the
    /// forward pass ran on; inference() is the forward pass that goes with this). No counterpart in the reference, whose
    /// backward_pass reads interm_forw (include/network/SwiftNetMLP.h:199-257); same values.
    std::vector<tnn::event> backward_pass_recompute(const DeviceMatrixView<T> input, const DeviceMatrixView<T> dL_doutput, DeviceMatricesView<T> output,
                                                    DeviceMatrixView<T> *dL_dinput = nullptr) {
        RequireDense(input);
        RequireDense(dL_doutput);
        if (dL_dinput != nullptr) RequireDense(*dL_dinput);
        if (input.m() != dL_doutput.m()) throw std::invalid_argument("input and dL_doutput differ in their number of rows.");
        const tnn_mlp_desc d = desc();
        ReserveWorkspace(tnn_mlp_train_step_workspace_bytes(&d, input.m()));
        tnn::abi_check(tnn_mlp_backward_recompute(&d, this->prepared_forward(), this->prepared_backward(), input.GetPointer(), dL_doutput.GetPointer(),
                                                  output.GetMatrixPointer(0), 0, dL_dinput ? dL_dinput->GetPointer() : nullptr, input.m(), workspace_,
                                                  workspace_bytes_, this->get_queue().abi()));
        return {tnn::event(this->get_queue().get())};
    }

    /// Whether backward_with_grid runs for this grid.
    bool supports_grid_training(const tnn_grid_desc &grid) const {
        const tnn_mlp_desc d = desc();
        return Network<T>::get_input_width() == WIDTH && tnn_grid_mlp_train_supported(&grid, &d) == TNN_OK;
    }

    /// The backward pass of this network behind a grid encoding of `positions`, for `dL_doutput`: weight gradients into `output`
    /// (raw layout) and the table's gradient (fp32, overwritten) into `grad_table` when it is not null. Encoding and forward
    /// pass are formed again on chip; the encoded matrix is never stored (inference_with_grid is the forward pass that goes
    /// with this). Batches from 2^17 rows on are visited in cell order, as GridEncoding's own backward pass does.
    /// `positions_as_last_ordered`: the caller vouches that the contents of `positions` have not changed since the last call
    /// that put them in cell order (inference_with_grid or this); if that call was for this pointer, batch size and grid, its
    /// order is used again instead of being formed again (25 us at 2^18 points).
    std::vector<tnn::event> backward_with_grid(const tnn_grid_desc &grid, const void *table, const float *positions, const DeviceMatrixView<T> dL_doutput,
                                               DeviceMatricesView<T> output, float *grad_table, const bool positions_as_last_ordered = false) {
        RequireDense(dL_doutput);
        const size_t M = dL_doutput.m();
        const tnn_mlp_desc d = desc();
        ReserveWorkspace(tnn_grid_mlp_train_step_workspace_bytes(&grid, &d, M));
        const void *order = nullptr;
        if (M >= (size_t(1) << 17)) {
            if (!(positions_as_last_ordered && OrderIsOf(grid, positions, M))) OrderPoints(grid, positions, M);
            order = m_grid_order->data();
        }
        tnn::abi_check(tnn_grid_mlp_backward(&grid, &d, order ? nullptr : positions, order, table, this->prepared_forward(), this->prepared_backward(),
                                             dL_doutput.GetPointer(), output.GetMatrixPointer(0), 0, grad_table, 1, M, workspace_, workspace_bytes_,
                                             this->get_queue().abi()));
        return {tnn::event(this->get_queue().get())};
    }

    Activation get_activation() const { return m_activation; }
    Activation get_output_activation() const { return m_output_activation; }

  private:
    tnn_mlp_desc desc() const {
        tnn_mlp_desc d = this->weights_desc();
        d.activation = tnn::to_abi(m_activation);
        d.output_activation = tnn::to_abi(m_output_activation);
        return d;
    }

    /// The workspace grows to the largest request seen; growing waits for the work that may still use the old one.
    void ReserveWorkspace(const size_t need) {
        if (need <= workspace_bytes_) return;
        this->get_queue().wait();
        tnn::detail::device_free(workspace_);
        workspace_ = nullptr;
        workspace_bytes_ = 0;
        tnn::hip_check(hipMalloc(&workspace_, need), "hipMalloc");
        workspace_bytes_ = need;
    }

    static void RequireDense(const DeviceMatrixView<T> &v) {
        if (v.stride() != v.n()) throw std::invalid_argument("Only dense row-major matrices (stride == n) are supported.");
    }

    static bool Supported(Activation a) { return a == Activation::ReLU || a == Activation::None || a == Activation::Sigmoid; }

    void SanityCheck() const override {
        static_assert(WIDTH == 16 || WIDTH == 32 || WIDTH == 64 || WIDTH == 128);
        static_assert(std::is_same<T, tnn::bf16>::value || std::is_same<T, tnn::half>::value);
        if (!Supported(m_activation)) throw std::runtime_error("m_activation must be ReLU or None or Sigmoid for now.");
        if (!Supported(m_output_activation)) throw std::runtime_error("m_output_activation must be ReLU or None or Sigmoid for now.");
    }

    void SanityCheckInference(const DeviceMatrix<T> &input, DeviceMatrix<T> &output) const {
        if ((input.m() % 8) != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        if (input.n() != Network<T>::get_input_width())
            throw std::invalid_argument("Input array too small. Input n: " + std::to_string(input.n()) +
                                        " != input width " + std::to_string(Network<T>::get_input_width()));
        if (output.m() != input.m() || output.n() < Network<T>::get_output_width()) throw std::invalid_argument("Output array too small");
    }

    static std::string Shape(size_t m, size_t n) { return "(" + std::to_string(m) + ", " + std::to_string(n) + ")"; }

    void SanityCheckForward(const DeviceMatrix<T> &input, DeviceMatrices<T> &interm) const {
        if ((input.m() % 8) != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        if (input.n() != Network<T>::get_input_width())
            throw std::invalid_argument("Input array too small. Input n: " + std::to_string(input.n()) +
                                        " != input width " + std::to_string(Network<T>::get_input_width()));
        if (interm.input_m() != input.m() || interm.input_n() != input.n())
            throw std::invalid_argument("intermediate_output_forward dim wrong doesn't match input shape, expected: " +
                                        Shape(input.m(), input.n()) + " but got: " + Shape(interm.input_m(), interm.input_n()));
        if (interm.middle_m() != input.m() || interm.middle_n() != WIDTH)
            throw std::invalid_argument("intermediate_output_forward array too small for middle results, expected: " +
                                        Shape(input.m(), WIDTH) + " but got: " + Shape(interm.middle_m(), interm.middle_n()));
        if (interm.output_m() != input.m() || interm.output_n() != Network<T>::get_output_width())
            throw std::invalid_argument("intermediate_output_forward array too small for output, expected: " +
                                        Shape(input.m(), Network<T>::get_output_width()) + " but got: " +
                                        Shape(interm.output_m(), interm.output_n()));
        if (int(interm.GetNumberOfMatrices()) != Network<T>::get_n_hidden_layers() + 2)
            throw std::invalid_argument("Not enough matrices in intermediate_output_forward array, expected: " +
                                        std::to_string(Network<T>::get_n_hidden_layers() + 2) + " but got: " +
                                        std::to_string(interm.GetNumberOfMatrices()));
    }

    void SanityCheckBackward(const DeviceMatrix<T> &input, DeviceMatrices<T> &output, DeviceMatrices<T> &interm_bwd,
                             const DeviceMatrices<T> &interm_fwd) const {
        const size_t in_w = Network<T>::get_input_width(), out_w = Network<T>::get_output_width();
        if ((input.m() % 8) != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        if (input.m() != interm_fwd.input_m() || input.n() != out_w)
            throw std::invalid_argument("Input array in backward pass too small. Input shape: " + Shape(input.m(), input.n()) +
                                        " expected: " + Shape(interm_fwd.input_m(), out_w));
        if (interm_fwd.input_m() != input.m() || interm_fwd.middle_m() != input.m() || interm_fwd.output_m() != input.m())
            throw std::invalid_argument("Intermediate_output_forward m dimension mismatch. Expected: " + std::to_string(input.m()));
        if (interm_fwd.input_n() != in_w || interm_fwd.middle_n() != WIDTH || interm_fwd.output_n() != out_w)
            throw std::invalid_argument("Intermediate_output_forward n dimension mismatch. Expected: (" + std::to_string(in_w) + ", " +
                                        std::to_string(WIDTH) + ", " + std::to_string(out_w) + ")");
        if (int(interm_fwd.GetNumberOfMatrices()) != Network<T>::get_n_hidden_layers() + 2)
            throw std::invalid_argument("Not enough matrices in intermediate_output_forward array. Required: " +
                                        std::to_string(Network<T>::get_n_hidden_layers() + 2));
        if (interm_bwd.input_m() != input.m() || interm_bwd.middle_m() != input.m() || interm_bwd.output_m() != input.m())
            throw std::invalid_argument("Intermediate_output_backward m dimension mismatch. Expected: " + std::to_string(input.m()));
        if (interm_bwd.input_n() != WIDTH || interm_bwd.middle_n() != WIDTH || interm_bwd.output_n() != out_w)
            throw std::invalid_argument("Intermediate_output_backward n dimension mismatch. Expected: (" + std::to_string(WIDTH) + ", " +
                                        std::to_string(WIDTH) + ", " + std::to_string(out_w) + ")");
        if (int(interm_bwd.GetNumberOfMatrices()) != Network<T>::get_n_hidden_layers() + 1)
            throw std::invalid_argument("Not enough matrices in intermediate_output_backward array. Required: " +
                                        std::to_string(Network<T>::get_n_hidden_layers() + 1));
        if (output.input_m() != in_w || output.input_n() != WIDTH)
            throw std::invalid_argument("Output of backward pass too small for input. Expected: " + Shape(in_w, WIDTH));
        if (output.middle_m() != WIDTH || output.middle_n() != WIDTH)
            throw std::invalid_argument("Output of backward pass too small for middle. Expected: " + Shape(WIDTH, WIDTH));
        if (output.output_m() != WIDTH || output.output_n() != out_w)
            throw std::invalid_argument("Output of backward pass too small for output. Expected: " + Shape(WIDTH, out_w));
        if (int(output.GetNumberOfMatrices()) != Network<T>::get_n_hidden_layers() + 1)
            throw std::invalid_argument("Not enough matrices in output of backward pass. Required: " +
                                        std::to_string(Network<T>::get_n_hidden_layers() + 1));
    }

    Activation m_activation;
    Activation m_output_activation;
    void *workspace_ = nullptr;
    size_t workspace_bytes_ = 0;
    std::unique_ptr<DeviceMatrix<float>> m_grid_order; // the last large batch in cell order, and what it was the order of:
    const float *m_ordered_positions = nullptr;
    size_t m_ordered_rows = 0;
    tnn_grid_desc m_ordered_grid{};

    bool OrderIsOf(const tnn_grid_desc &grid, const float *positions, const size_t M) const {
        return m_grid_order && m_ordered_positions == positions && m_ordered_rows == M && std::memcmp(&m_ordered_grid, &grid, sizeof(grid)) == 0;
    }
    void OrderPoints(const tnn_grid_desc &grid, const float *positions, const size_t M) {
        const size_t bytes = tnn_grid_order_bytes(&grid, M);
        if (!m_grid_order || m_grid_order->size() * sizeof(float) < bytes)
            m_grid_order = std::make_unique<DeviceMatrix<float>>((bytes + sizeof(float) - 1) / sizeof(float), 1, this->get_queue());
        m_ordered_positions = nullptr; // (stays so if the call below throws)
        tnn::abi_check(tnn_grid_order_points(&grid, positions, M, m_grid_order->data(), m_grid_order->size() * sizeof(float), this->get_queue().abi()));
        m_ordered_positions = positions;
        m_ordered_rows = M;
        m_ordered_grid = grid;
    }
};

template <typename T, int WIDTH>
std::shared_ptr<SwiftNetMLP<T, WIDTH>> create_network(tnn::queue &q, const int output_width, const int n_hidden_layers, Activation activation,
                                                      Activation output_activation) {
    return std::make_shared<SwiftNetMLP<T, WIDTH>>(q, WIDTH, output_width, n_hidden_layers, activation, output_activation);
}
