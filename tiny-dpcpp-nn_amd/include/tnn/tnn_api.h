// The tensor-level module interface that the Python bindings wrap. Mirrors include/tnn_api.h of the reference:
// tnn::Module (:62-303), EncodingModule<T> (:306-474), NetworkModule<T, WIDTH> (:477-697). Tensors are
// PyTorch-ROCm tensors on the GPU; every method runs on torch's current HIP stream at the time of the call (the
// reference takes the current XPU stream's queue, :295-302). Results are handed back as fresh torch allocations; the
// work is ordered with the caller's tensor operations by the stream, so no method makes the host wait.
#pragma once

#include <c10/hip/HIPStream.h>
#include <torch/torch.h>

#include <tuple>

#include "SwiftNetMLP.h"
#include "encoding_factory.h"
#include "io.h"

#define CHECK_GPU(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a GPU tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x)                                                                                                 \
    CHECK_GPU(x);                                                                                                      \
    CHECK_CONTIGUOUS(x)

namespace tnn {

using fp16 = tnn::half;

template <typename T> struct torch_type {};
template <> struct torch_type<int> { static constexpr auto dtype = torch::kInt32; };
template <> struct torch_type<double> { static constexpr auto dtype = torch::kFloat64; };
template <> struct torch_type<float> { static constexpr auto dtype = torch::kFloat32; };
template <> struct torch_type<fp16> { static constexpr auto dtype = c10::ScalarType::Half; };
template <> struct torch_type<bf16> { static constexpr auto dtype = c10::ScalarType::BFloat16; };

class Module {
  public:
    Module() : queue_(c10::hip::getCurrentHIPStream().stream()), device_index_(c10::hip::current_device()) {}
    virtual ~Module() {}

    virtual torch::Tensor initialize_params() = 0;
    virtual torch::Tensor initialize_params(const torch::Tensor &tensor) = 0;
    virtual void set_params(const torch::Tensor &tensor, bool weights_are_packed) = 0;
    virtual torch::Tensor get_params() = 0;
    virtual torch::Tensor forward_pass(const torch::Tensor &input_tensor) = 0;
    virtual std::tuple<torch::Tensor, torch::Tensor> backward_pass(const torch::Tensor &input_tensor, const torch::Tensor &input_from_fwd,
                                                                   bool pack_transpose_gradient, bool get_dl_dinput) = 0;
    virtual std::tuple<torch::Tensor, torch::Tensor> backward_pass(const torch::Tensor &input_tensor, bool pack_transpose_gradient,
                                                                   bool get_dl_dinput) = 0;
    virtual torch::Tensor inference(const torch::Tensor &input_tensor) = 0;
    virtual size_t n_params() = 0;
    virtual size_t n_output_dims() = 0;

    /// Encoding modules whose encoding is a grid: its descriptor and its table on the device (nullptr otherwise).
    virtual const tnn_grid_desc *grid_descriptor() const { return nullptr; }
    virtual const void *grid_table() const { return nullptr; }
    /// Network modules: inference on `encoding`'s output for `positions`, in one kernel, when can_fuse_encoding says so.
    /// No counterpart in the reference (NetworkWithInputEncoding runs the two modules in turn,
    /// dpcpp_bindings/tiny_dpcpp_nn/modules.py:357-421); the values are those of the two calls.
    virtual bool can_fuse_encoding(const Module &) const { return false; }
    virtual torch::Tensor inference_with_encoding(const Module &, const torch::Tensor &, bool = false) {
        throw std::runtime_error("inference_with_encoding: not a network module");
    }

    /// Network modules, training without stored activations (no counterpart in the reference, whose forward_pass keeps
    /// interm_forw for backward_pass, include/tnn_api.h:541-603): when can_recompute_backward() holds, a training step may run
    /// inference() as its forward pass and backward_pass_recompute(grad_output, the same input, ...) as its backward pass; the
    /// activations are formed again on chip. Same return value as backward_pass.
    virtual bool can_recompute_backward() const { return false; }
    virtual std::tuple<torch::Tensor, torch::Tensor> backward_pass_recompute(const torch::Tensor &, const torch::Tensor &, bool, bool) {
        throw std::runtime_error("backward_pass_recompute: not available for this module");
    }
    /// The same behind a grid encoding: inference_with_encoding() is the forward pass, backward_with_encoding returns the
    /// network's weight gradients (packed on request) and the gradient of the encoding's table.
    virtual bool can_train_with_encoding(const Module &) const { return false; }
    virtual std::tuple<torch::Tensor, torch::Tensor> backward_with_encoding(const Module &, const torch::Tensor &, const torch::Tensor &, bool, bool = false) {
        throw std::runtime_error("backward_with_encoding: not a network module");
    }

    tnn::queue &get_queue() { return queue_; }

    /// First thing in every method: the module's kernels go to the stream the caller's tensor operations are on, so inputs
    /// produced there are complete when the kernels read them and the tensors handed back (allocated from that stream's
    /// pool) are written on it. When the caller has changed streams since the last call, the new stream first waits for
    /// what the module still has in flight on the old one (its workspaces and parameter copies are shared between calls).
    void enter() {
        const hipStream_t now = c10::hip::getCurrentHIPStream(device_index_).stream();
        const hipStream_t before = queue_.get();
        if (now == before) return;
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        (void)hipStreamIsCapturing(now, &capturing);
        if (capturing == hipStreamCaptureStatusNone) {
            hipEvent_t done = nullptr;
            tnn::hip_check(hipEventCreateWithFlags(&done, hipEventDisableTiming), "hipEventCreateWithFlags");
            tnn::hip_check(hipEventRecord(done, before), "hipEventRecord");
            tnn::hip_check(hipStreamWaitEvent(now, done, 0), "hipStreamWaitEvent");
            tnn::hip_check(hipEventDestroy(done), "hipEventDestroy"); // released once it has completed
        }
        queue_.rebind(now);
    }

    /// Nothing to wait for: the call's work is on the caller's stream (the reference blocks here).
    void finish() {}

    template <typename T> static std::vector<T> convertTensorToVector(const torch::Tensor &tensor) {
        const auto cpu = tensor.to(torch::kCPU).to(torch::kFloat32).contiguous();
        const float *begin = cpu.data_ptr<float>();
        std::vector<T> result;
        result.reserve(cpu.numel());
        for (int64_t i = 0; i < cpu.numel(); ++i) result.push_back(T(begin[i]));
        return result;
    }

    template <typename T> torch::Tensor convertVectorToTensor(const std::vector<T> &v) const {
        std::vector<float> f(v.begin(), v.end());
        return torch::from_blob(f.data(), {(int64_t)f.size()}, torch::TensorOptions().dtype(torch::kFloat32)).clone().to(device());
    }

    /// Fresh tensor holding a copy of device memory owned by the module.
    template <typename T> torch::Tensor fromDevice(T *ptr, std::initializer_list<int64_t> sizes) const {
        return torch::from_blob(ptr, sizes, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device())).clone();
    }
    template <typename T> torch::Tensor convertDeviceMatrixViewToTorchTensor(const DeviceMatrixView<T> &dm) const {
        return fromDevice<T>(dm.GetPointer(), {(int64_t)dm.m(), (int64_t)dm.n()});
    }
    template <typename T> torch::Tensor convertDeviceMatrixToTorchTensor(DeviceMatrix<T> &dm) const {
        return fromDevice<T>(dm.data(), {(int64_t)dm.rows(), (int64_t)dm.cols()});
    }
    template <typename T> torch::Tensor convertDeviceMatricesToTorchTensor(const DeviceMatrices<T> &dm) const {
        return fromDevice<T>(dm.GetViews().GetMatrixPointer(0), {(int64_t)dm.nelements(), 1});
    }

  protected:
    virtual void FreeWorkspace() = 0;
    virtual void AllocateWorkspace(const size_t batch_size) = 0;
    c10::Device device() const { return c10::Device(c10::DeviceType::CUDA, device_index_); }

  private:
    tnn::queue queue_;
    c10::DeviceIndex device_index_;
};

/************************************************ENCODING MODULE */
template <typename T> class EncodingModule : public Module {
  public:
    EncodingModule(std::string filename, std::optional<uint32_t> padded_output_width = std::nullopt)
        : max_batch_size_(0), output_encoding_ptr_(nullptr) {
        encoding_ = create_encoding<T>(io::loadJsonConfig(filename), this->get_queue(), padded_output_width);
        initialize_ptr();
    }

    EncodingModule(const json &encoding_config, std::optional<uint32_t> padded_output_width = std::nullopt)
        : max_batch_size_(0), output_encoding_ptr_(nullptr) {
        encoding_ = create_encoding<T>(io::validateAndCopyEncodingConfig(encoding_config), this->get_queue(), padded_output_width);
        initialize_ptr();
    }

    ~EncodingModule() { this->FreeWorkspace(); }

    torch::Tensor forward_pass(const torch::Tensor &input_tensor) override {
        this->enter();
        CHECK_INPUT(input_tensor);
        TORCH_CHECK(input_tensor.scalar_type() == torch::kFloat32, "input_tensor must be float32");
        const size_t batch_size = input_tensor.sizes()[0];
        if (input_tensor.sizes().size() != 2 || input_tensor.sizes()[1] != encoding_->get_input_width())
            throw std::runtime_error("Input tensor has incorrect dimensions");
        const uint32_t out_w = encoding_->get_padded_output_width();
        if (batch_size == 0) return torch::empty({0, (int64_t)out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));

        DeviceMatrixView<float> input_dmv(batch_size, encoding_->get_input_width(), encoding_->get_input_width(), input_tensor.data_ptr<float>());
        // the kernel writes the tensor that is handed back (a fresh allocation as the reference's clone is, without the copy)
        torch::Tensor output = torch::empty({(int64_t)batch_size, (int64_t)out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatrixView<T> output_encoding(batch_size, out_w, out_w, reinterpret_cast<T *>(output.data_ptr()));
        std::unique_ptr<Context> model_ctx = encoding_->forward_impl(input_dmv, &output_encoding);
        this->finish();
        return output;
    }

    torch::Tensor inference(const torch::Tensor &input_tensor) override { return forward_pass(input_tensor); }

    std::tuple<torch::Tensor, torch::Tensor> backward_pass(const torch::Tensor &, bool = false, bool = false) override {
        throw std::runtime_error("backward_pass needs input_from_fwd");
    }

    std::tuple<torch::Tensor, torch::Tensor> backward_pass(const torch::Tensor &grad_output, const torch::Tensor &input_from_fwd,
                                                           bool pack_transpose_gradient = false, bool get_dl_dinput = false) override {
        this->enter();
        if (encoding_->get_n_params() == 0) return {torch::Tensor(), torch::Tensor()};
        CHECK_INPUT(grad_output);
        CHECK_INPUT(input_from_fwd);
        if (pack_transpose_gradient) throw std::invalid_argument("Encoding params are not packed");
        if (get_dl_dinput) throw std::invalid_argument("Encoding get_dl_dinput not implemented");
        TORCH_CHECK(grad_output.scalar_type() == torch_type<T>::dtype, "grad_output has the wrong dtype");
        TORCH_CHECK(input_from_fwd.scalar_type() == torch::kFloat32, "input_from_fwd must be float32");

        const int64_t batch_size = grad_output.sizes()[0];
        const int64_t input_width = encoding_->get_input_width();
        const auto input_sizes = input_from_fwd.sizes();
        if (input_sizes.size() != 2 || input_sizes[0] != batch_size || input_sizes[1] != input_width)
            throw std::runtime_error("Size mismatch for input_from_fwd: expected [" + std::to_string(batch_size) + ", " +
                                     std::to_string(input_width) + "], but got [" + std::to_string(input_sizes[0]) + ", " +
                                     std::to_string(input_sizes.size() > 1 ? input_sizes[1] : 0) + "]");
        if (grad_output.sizes().size() != 2 || grad_output.sizes()[1] != encoding_->get_padded_output_width())
            throw std::runtime_error("grad_output must be [batch, padded output width]");

        const uint32_t out_w = encoding_->get_padded_output_width();
        DeviceMatrixView<T> dL_doutput_dmv(batch_size, out_w, out_w, reinterpret_cast<T *>(grad_output.data_ptr()));
        DeviceMatrixView<float> input_encoding_dmv(batch_size, input_width, input_width, input_from_fwd.data_ptr<float>());
        // the scatter overwrites its whole destination: it is the tensor that is handed back; the module keeps a reference
        // for get_encoding_grads
        last_gradients_ = torch::empty({(int64_t)encoding_->get_n_params(), 1}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatrixView<T> gradients_view(encoding_->get_n_params(), 1, 1, reinterpret_cast<T *>(last_gradients_.data_ptr()));
        Context ctx;
        encoding_->backward_impl(ctx, input_encoding_dmv, dL_doutput_dmv, &gradients_view);
        this->finish();
        return {torch::Tensor(), last_gradients_};
    }

    torch::Tensor initialize_params() override { return get_params(); }
    torch::Tensor initialize_params(const torch::Tensor &tensor) override {
        this->enter();
        set_params(tensor, false);
        return get_params();
    }

    void set_params(const torch::Tensor &params, bool weights_are_packed) override {
        this->enter();
        if (encoding_->get_params() == nullptr) throw std::runtime_error("no encoding params to set");
        if (weights_are_packed) throw std::runtime_error("Packed weights are not supported in api set params");
        CHECK_INPUT(params);
        TORCH_CHECK((size_t)params.numel() == encoding_->get_n_params(), "params has ", params.numel(), " elements, the encoding has ",
                    encoding_->get_n_params());
        TORCH_CHECK(params.scalar_type() == torch_type<T>::dtype, "params has the wrong dtype");
        // No copy: from now on the table IS the caller's tensor (a reference keeps it alive), so later writes to it by any
        // route are seen by the kernels, and pushing the same tensor again costs nothing. The reference copies, through the
        // host (include/tnn_api.h:430-446); get_params() hands back a copy either way.
        if (!table_alias_.defined() || table_alias_.data_ptr() != params.data_ptr()) {
            encoding_->adopt_params(std::make_shared<DeviceMatrix<T>>(encoding_->get_n_params(), 1, this->get_queue(), params.data_ptr<T>()));
            table_alias_ = params;
        }
    }

    torch::Tensor get_params() override {
        this->enter();
        if (encoding_->get_params()) return convertDeviceMatrixToTorchTensor<T>(*encoding_->get_params());
        return torch::empty({0});
    }

    size_t n_params() override { return encoding_->get_n_params(); }
    size_t n_output_dims() override { return encoding_->get_padded_output_width(); }
    const tnn_grid_desc *grid_descriptor() const override {
        const auto *grid = dynamic_cast<const tinydpcppnn::encodings::grid::GridEncodingTemplated<T> *>(encoding_.get());
        return grid ? &grid->descriptor() : nullptr;
    }
    const void *grid_table() const override { return grid_descriptor() ? encoding_->get_params()->data() : nullptr; }
    std::vector<T> get_encoding_params() { return encoding_->get_params()->copy_to_host(); }
    /// The gradients of the last backward_pass (zeros before the first one).
    std::vector<T> get_encoding_grads() {
        if (!last_gradients_.defined()) return std::vector<T>(encoding_->get_n_params(), T(0));
        return convertTensorToVector<T>(last_gradients_);
    }

  protected:
    void FreeWorkspace() override {
        tnn::detail::device_free(output_encoding_ptr_);
        output_encoding_ptr_ = nullptr;
        max_batch_size_ = 0;
    }

    void AllocateWorkspace(const size_t batch_size) override {
        if (batch_size > max_batch_size_) {
            this->get_queue().wait();
            this->FreeWorkspace();
            output_encoding_ptr_ = tnn::detail::device_alloc<T>(batch_size * encoding_->get_padded_output_width());
            max_batch_size_ = batch_size;
        }
    }

  private:
    void initialize_ptr() {}

    std::shared_ptr<Encoding<T>> encoding_;
    torch::Tensor table_alias_; // the tensor whose memory is the encoding's table, once set_params has been called
    torch::Tensor last_gradients_;
    size_t max_batch_size_; // the workspace fits every batch size seen so far
    T *output_encoding_ptr_;
};

/**************************************NETWORK MODULE */
template <typename T, int WIDTH> class NetworkModule : public Module {
  public:
    NetworkModule(const int input_width, const int output_width, const int n_hidden_layers, const Activation activation,
                  const Activation output_activation, bool use_bias)
        : network_(this->get_queue(), input_width, output_width, n_hidden_layers, activation, output_activation,
                   Network<T>::WeightInitMode::xavier_normal, use_bias),
          net_gradients_(network_.get_n_hidden_layers() + 1, network_.get_network_width(), WIDTH, WIDTH, WIDTH, WIDTH,
                         network_.get_output_width(), this->get_queue()),
          net_gradients_packed_(network_.get_n_hidden_layers() + 1, network_.get_network_width(), WIDTH, WIDTH, WIDTH, WIDTH,
                                network_.get_output_width(), this->get_queue()),
          max_batch_size_(0), interm_forw_ptr_(nullptr), interm_backw_ptr_(nullptr), dL_dinput_ptr_(nullptr) {
        net_gradients_.fill(T(0.0f)).wait();
    }

    ~NetworkModule() { this->FreeWorkspace(); }

    torch::Tensor inference(const torch::Tensor &input_tensor) override {
        this->enter();
        const size_t batch_size = CheckedBatch(input_tensor, network_.get_input_width());
        const int64_t out_w = network_.get_output_width();
        if (batch_size == 0) return torch::empty({0, out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatrixView<T> input_dm(batch_size, network_.get_input_width(), network_.get_input_width(),
                                     reinterpret_cast<T *>(input_tensor.data_ptr()));
        // the kernel writes the tensor that is handed back: a fresh allocation, as the reference's clone is, without the copy
        torch::Tensor output = torch::empty({(int64_t)batch_size, out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatricesView<T> output_network(1, batch_size, network_.get_output_width(), 0, 0, 0, 0, reinterpret_cast<T *>(output.data_ptr()));
        network_.inference(input_dm, output_network, {});
        this->finish();
        return output;
    }

    bool can_fuse_encoding(const Module &encoding) const override {
        const tnn_grid_desc *grid = encoding.grid_descriptor();
        return grid && network_.supports_grid_input(*grid);
    }

    /// a_backward_pass_follows: this is the forward pass of a training step (the batch is then put in cell order from the
    /// size on from which backward_with_encoding would order it, which can take the order over).
    torch::Tensor inference_with_encoding(const Module &encoding, const torch::Tensor &positions, bool a_backward_pass_follows = false) override {
        this->enter();
        const tnn_grid_desc *grid = encoding.grid_descriptor();
        if (!grid || !network_.supports_grid_input(*grid))
            throw std::invalid_argument("inference_with_encoding: this encoding / network pair runs as two calls (" +
                                        std::string(tnn_last_error()) + ")");
        CHECK_INPUT(positions);
        TORCH_CHECK(positions.dim() == 2 && positions.scalar_type() == torch::kFloat32, "positions must be a float32 matrix");
        if (positions.sizes()[1] != (int64_t)grid->n_dims) throw std::runtime_error("Input tensor has incorrect dimensions");
        if (positions.sizes()[0] % 8 != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        const size_t batch_size = positions.sizes()[0];
        const int64_t out_w = network_.get_output_width();
        if (batch_size == 0) return torch::empty({0, out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        torch::Tensor output = torch::empty({(int64_t)batch_size, out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatricesView<T> output_network(1, batch_size, network_.get_output_width(), 0, 0, 0, 0, reinterpret_cast<T *>(output.data_ptr()));
        network_.inference_with_grid(*grid, encoding.grid_table(), positions.data_ptr<float>(), batch_size, output_network, a_backward_pass_follows);
        this->finish();
        return output;
    }

    torch::Tensor forward_pass(const torch::Tensor &input_tensor) override {
        this->enter();
        const size_t batch_size = CheckedBatch(input_tensor, network_.get_input_width());
        const int64_t out_w = network_.get_output_width();
        if (batch_size == 0) return torch::empty({0, out_w}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatrixView<T> input_dm(batch_size, network_.get_input_width(), network_.get_input_width(),
                                     reinterpret_cast<T *>(input_tensor.data_ptr()));
        this->AllocateWorkspace(batch_size);
        DeviceMatricesView<T> output_network = ForwardViews(batch_size);
        network_.forward_pass(input_dm, output_network, {});
        this->finish();
        forward_batch_size_ = batch_size;
        return fromDevice<T>(output_network.GetMatrixPointer(network_.get_n_hidden_layers() + 1), {(int64_t)batch_size, out_w});
    }

    std::tuple<torch::Tensor, torch::Tensor> backward_pass(const torch::Tensor &, const torch::Tensor &, bool, bool) override {
        throw std::runtime_error("backward_pass of NetworkModule takes no input_from_fwd");
    }

    std::tuple<torch::Tensor, torch::Tensor> backward_pass(const torch::Tensor &grad_output, bool pack_transpose_gradient,
                                                           bool get_dl_dinput) override {
        this->enter();
        CHECK_INPUT(grad_output);
        TORCH_CHECK(grad_output.dim() == 2, "grad_output must have two dimensions");
        TORCH_CHECK(grad_output.scalar_type() == torch_type<T>::dtype, "grad_output has the wrong dtype");
        const size_t batch_size = grad_output.sizes()[0];
        if (grad_output.size(1) != network_.get_output_width())
            throw std::invalid_argument("grad_output.size(1): " + std::to_string(grad_output.size(1)) +
                                        " is not equal to  get_padded_output_width" + std::to_string(network_.get_output_width()));
        if (batch_size % 8 != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        // The activations of the last forward_pass are the other operand; they live in the module's workspace.
        if (batch_size == 0 || batch_size != forward_batch_size_)
            throw std::invalid_argument("backward_pass: batch size " + std::to_string(batch_size) +
                                        " does not match the last forward_pass (" + std::to_string(forward_batch_size_) + ")");

        DeviceMatrixView<T> dL_doutput(batch_size, network_.get_output_width(), network_.get_output_width(),
                                       reinterpret_cast<T *>(grad_output.data_ptr()));
        DeviceMatricesView<T> interm_bwd(network_.get_n_hidden_layers() + 1, batch_size, network_.get_input_width(), batch_size,
                                         network_.get_network_width(), batch_size, network_.get_output_width(), interm_backw_ptr_);
        DeviceMatricesView<T> interm_fwd = ForwardViews(batch_size);
        // dL/dinput goes straight into the tensor that is handed back
        torch::Tensor input_grad;
        if (get_dl_dinput)
            input_grad = torch::empty({(int64_t)(batch_size * network_.get_input_width()), 1},
                                      torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatrixView<T> dL_dinput(batch_size, network_.get_input_width(), network_.get_input_width(),
                                      get_dl_dinput ? reinterpret_cast<T *>(input_grad.data_ptr()) : dL_dinput_ptr_);

        network_.backward_pass(dL_doutput, net_gradients_.GetViews(), interm_bwd, interm_fwd, {}, get_dl_dinput ? &dL_dinput : nullptr);
        this->finish();

        // Pack and transpose: the kernels compute x * W, torch-style gradients are laid out for W * x. The reference does it in
        // place (through a temporary); here the packed copy has a buffer of its own, so nothing is allocated per call.
        const DeviceMatrices<T> *result = &net_gradients_;
        if (pack_transpose_gradient) {
            net_gradients_.PackAndTranspose(net_gradients_packed_);
            this->finish();
            result = &net_gradients_packed_;
        }

        return {input_grad, fromDevice<T>(result->GetViews().GetMatrixPointer(0), {(int64_t)result->nelements(), 1})};
    }

    bool can_recompute_backward() const override { return network_.supports_backward_recompute(); }

    std::tuple<torch::Tensor, torch::Tensor> backward_pass_recompute(const torch::Tensor &grad_output, const torch::Tensor &input_tensor,
                                                                     bool pack_transpose_gradient, bool get_dl_dinput) override {
        this->enter();
        const size_t batch_size = CheckedBatch(input_tensor, network_.get_input_width());
        CheckedGradOutput(grad_output, batch_size);
        if (batch_size == 0) throw std::invalid_argument("backward_pass_recompute: empty batch");
        DeviceMatrixView<T> input_dm(batch_size, network_.get_input_width(), network_.get_input_width(), reinterpret_cast<T *>(input_tensor.data_ptr()));
        DeviceMatrixView<T> dL_doutput(batch_size, network_.get_output_width(), network_.get_output_width(), reinterpret_cast<T *>(grad_output.data_ptr()));
        torch::Tensor input_grad;
        if (get_dl_dinput)
            input_grad = torch::empty({(int64_t)(batch_size * network_.get_input_width()), 1}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        DeviceMatrixView<T> dL_dinput(batch_size, network_.get_input_width(), network_.get_input_width(),
                                      get_dl_dinput ? reinterpret_cast<T *>(input_grad.data_ptr()) : nullptr);
        network_.backward_pass_recompute(input_dm, dL_doutput, net_gradients_.GetViews(), get_dl_dinput ? &dL_dinput : nullptr);
        return {input_grad, GradientsTensor(pack_transpose_gradient)};
    }

    bool can_train_with_encoding(const Module &encoding) const override {
        const tnn_grid_desc *grid = encoding.grid_descriptor();
        return grid && network_.supports_grid_input(*grid) && network_.supports_grid_training(*grid);
    }

    std::tuple<torch::Tensor, torch::Tensor> backward_with_encoding(const Module &encoding, const torch::Tensor &positions,
                                                                    const torch::Tensor &grad_output, bool pack_transpose_gradient,
                                                                    bool positions_unchanged_since_forward = false) override {
        this->enter();
        const tnn_grid_desc *grid = encoding.grid_descriptor();
        if (!grid || !network_.supports_grid_training(*grid))
            throw std::invalid_argument("backward_with_encoding: this encoding / network pair trains as two modules (" + std::string(tnn_last_error()) + ")");
        CHECK_INPUT(positions);
        TORCH_CHECK(positions.dim() == 2 && positions.scalar_type() == torch::kFloat32, "positions must be a float32 matrix");
        if (positions.sizes()[1] != (int64_t)grid->n_dims) throw std::runtime_error("Input tensor has incorrect dimensions");
        const size_t batch_size = positions.sizes()[0];
        if (batch_size == 0 || batch_size % 8 != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        CheckedGradOutput(grad_output, batch_size);
        DeviceMatrixView<T> dL_doutput(batch_size, network_.get_output_width(), network_.get_output_width(), reinterpret_cast<T *>(grad_output.data_ptr()));
        // the scatter overwrites its whole destination: it is the tensor that is handed back
        torch::Tensor table_grad = torch::empty({(int64_t)tnn_grid_n_params(grid), 1}, torch::TensorOptions().dtype(torch::kFloat32).device(device()));
        network_.backward_with_grid(*grid, encoding.grid_table(), positions.data_ptr<float>(), dL_doutput, net_gradients_.GetViews(),
                                    table_grad.data_ptr<float>(), positions_unchanged_since_forward);
        return {GradientsTensor(pack_transpose_gradient), table_grad};
    }

    torch::Tensor initialize_params() override { return get_params(); }
    torch::Tensor get_params() override {
        this->enter();
        return convertDeviceMatricesToTorchTensor(network_.get_weights_matrices());
    }
    torch::Tensor initialize_params(const torch::Tensor &tensor) override {
        this->enter();
        set_params(tensor, false);
        return initialize_params();
    }

    size_t n_params() override { return network_.get_weights_matrices().nelements(); }
    size_t n_output_dims() override { return network_.get_output_width(); }

    /// The parameters stay on the device: a GPU tensor of any floating dtype is converted and (if unpacked)
    /// packed there. A CPU tensor takes the reference's route through a host vector.
    void set_params(const torch::Tensor &params, bool weights_are_packed) override {
        this->enter();
        if ((size_t)params.numel() != n_params())
            throw std::runtime_error("m_weights_matrices nelements: " + std::to_string(n_params()) +
                                     " does not match unpacked_weights size: " + std::to_string(params.numel()) +
                                     ". Consider padding input and output to have the same amount as network_width");
        if (!params.device().is_cuda()) {
            network_.set_weights_matrices(convertTensorToVector<T>(params), weights_are_packed);
            return;
        }
        const torch::Tensor p = params.contiguous();
        switch (p.scalar_type()) {
        case torch::kFloat32: network_.set_weights_matrices_from_device(p.data_ptr<float>(), weights_are_packed); break;
        case c10::ScalarType::Half:
            network_.set_weights_matrices_from_device(reinterpret_cast<const fp16 *>(p.data_ptr()), weights_are_packed);
            break;
        case c10::ScalarType::BFloat16:
            network_.set_weights_matrices_from_device(reinterpret_cast<const bf16 *>(p.data_ptr()), weights_are_packed);
            break;
        default: throw std::invalid_argument("params must be float32, float16 or bfloat16");
        }
    }

    std::vector<T> get_network_params() { return network_.get_weights_matrices().copy_to_host(); }
    std::vector<T> get_network_grads() { return net_gradients_.copy_to_host(); } // raw layout

  protected:
    void AllocateWorkspace(const size_t batch_size) override {
        if (batch_size > max_batch_size_) {
            this->get_queue().wait();
            this->FreeWorkspace();
            const size_t in_w = network_.get_input_width(), out_w = network_.get_output_width(), w = network_.get_network_width(),
                         l = network_.get_n_hidden_layers();
            interm_forw_ptr_ = tnn::detail::device_alloc<T>(batch_size * (in_w + out_w + w * l));
            interm_backw_ptr_ = tnn::detail::device_alloc<T>(batch_size * (out_w + w * l));
            dL_dinput_ptr_ = tnn::detail::device_alloc<T>(batch_size * in_w);
            max_batch_size_ = batch_size;
        }
    }

    void FreeWorkspace() override {
        tnn::detail::device_free(interm_forw_ptr_);
        interm_forw_ptr_ = nullptr;
        tnn::detail::device_free(interm_backw_ptr_);
        interm_backw_ptr_ = nullptr;
        tnn::detail::device_free(dL_dinput_ptr_);
        dL_dinput_ptr_ = nullptr;
        max_batch_size_ = 0;
        forward_batch_size_ = 0;
    }

  private:
    size_t CheckedBatch(const torch::Tensor &input_tensor, const uint32_t width) const {
        CHECK_INPUT(input_tensor);
        TORCH_CHECK(input_tensor.dim() == 2, "input_tensor must have two dimensions");
        TORCH_CHECK(input_tensor.scalar_type() == torch_type<T>::dtype, "input_tensor has the wrong dtype");
        if (input_tensor.sizes()[1] != width)
            throw std::invalid_argument("Input array too small. Input n: " + std::to_string(input_tensor.sizes()[1]) + " != input width " +
                                        std::to_string(width));
        if (input_tensor.sizes()[0] % 8 != 0) throw std::invalid_argument("Batch size is not divisible by 8.");
        return input_tensor.sizes()[0];
    }

    void CheckedGradOutput(const torch::Tensor &grad_output, const size_t batch_size) const {
        CHECK_INPUT(grad_output);
        TORCH_CHECK(grad_output.dim() == 2, "grad_output must have two dimensions");
        TORCH_CHECK(grad_output.scalar_type() == torch_type<T>::dtype, "grad_output has the wrong dtype");
        if (grad_output.size(1) != network_.get_output_width())
            throw std::invalid_argument("grad_output.size(1): " + std::to_string(grad_output.size(1)) +
                                        " is not equal to  get_padded_output_width" + std::to_string(network_.get_output_width()));
        if ((size_t)grad_output.size(0) != batch_size)
            throw std::invalid_argument("grad_output has " + std::to_string(grad_output.size(0)) + " rows, the forward pass had " + std::to_string(batch_size));
    }

    /// The raw gradients the last backward pass left in net_gradients_, as a fresh tensor: a copy, or (packed) the output of the
    /// pack-and-transpose kernel, which writes the tensor directly.
    torch::Tensor GradientsTensor(const bool packed) {
        const int64_t n = (int64_t)net_gradients_.nelements();
        torch::Tensor out = torch::empty({n, 1}, torch::TensorOptions().dtype(torch_type<T>::dtype).device(device()));
        if (packed)
            tnn::abi_check(tnn_pack_and_transpose(tnn::dtype_of<T>::value, WIDTH, network_.get_n_hidden_layers() + 1, net_gradients_.data(), out.data_ptr(),
                                                  this->get_queue().abi()));
        else
            tnn::hip_check(hipMemcpyAsync(out.data_ptr(), net_gradients_.data(), (size_t)n * sizeof(T), hipMemcpyDeviceToDevice, this->get_queue().get()),
                           "hipMemcpyAsync");
        return out;
    }

    DeviceMatricesView<T> ForwardViews(const size_t batch_size) const {
        return DeviceMatricesView<T>(network_.get_n_hidden_layers() + 2, batch_size, network_.get_input_width(), batch_size,
                                     network_.get_network_width(), batch_size, network_.get_output_width(), interm_forw_ptr_);
    }

    SwiftNetMLP<T, WIDTH> network_;
    DeviceMatrices<T> net_gradients_; // independent of the batch size; raw [out][in] as the backward pass writes them
    DeviceMatrices<T> net_gradients_packed_; // the same in the parameter layout
    size_t max_batch_size_;           // the workspaces fit every batch size seen so far
    size_t forward_batch_size_ = 0;   // batch size of the activations held in interm_forw_ptr_
    T *interm_forw_ptr_;
    T *interm_backw_ptr_;
    T *dL_dinput_ptr_;
};

} // namespace tnn
