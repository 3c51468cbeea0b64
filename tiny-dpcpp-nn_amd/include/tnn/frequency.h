// Frequency encoding: every input feature becomes sin / cos pairs at n_frequencies octaves, padded with ones. Mirrors
// include/encodings/frequency.h:20-146 of the reference, including the ForwardContext that keeps dy/dx for the backward
// pass when input gradients were asked for.
#pragma once

#include "encoding.h"

template <typename T> class FrequencyEncoding : public Encoding<T> {
  public:
    FrequencyEncoding(const uint32_t n_frequencies, const uint32_t n_dims_to_encode, const uint32_t padded_output_width, tnn::queue &Q)
        : Encoding<T>(n_dims_to_encode, n_dims_to_encode * n_frequencies * 2, padded_output_width, Q), n_frequencies_{n_frequencies} {}

    std::unique_ptr<Context> forward_impl(const DeviceMatrixView<float> input, DeviceMatrixView<T> *output = nullptr,
                                          bool use_inference_params = false, bool prepare_input_gradients = false) override {
        if (!output) return std::make_unique<Context>();
        if (input.n() != this->get_input_width()) throw std::invalid_argument("input dimensions do not coincide with encoder");
        if (use_inference_params) throw std::invalid_argument("Cannot yet use inference params");
        if (output->m() != input.m()) throw std::invalid_argument("Differing row numbers");
        if (output->n() != this->get_padded_output_width()) throw std::invalid_argument("number of cols has to be padded output width.");
        if (input.stride() != input.n() || output->stride() != output->n()) throw std::invalid_argument("Only dense matrices are supported.");

        std::unique_ptr<Context> forward = std::make_unique<Context>();
        float *dy_dx = nullptr;
        if (prepare_input_gradients) {
            auto ctx = std::make_unique<ForwardContext>(input.m(), this->get_output_width(), this->get_queue());
            dy_dx = ctx->dy_dx.data();
            forward = std::move(ctx);
        }
        tnn::abi_check(tnn_frequency_forward(input.GetPointer(), this->get_input_width(), n_frequencies_, output->GetPointer(),
                                             tnn::dtype_of<T>::value, this->get_padded_output_width(), dy_dx, input.m(),
                                             this->get_queue().abi()));
        return forward;
    }

    void backward_impl(const Context &ctx, const DeviceMatrixView<float> input, const DeviceMatrixView<T> dL_doutput,
                       DeviceMatrixView<T> * = nullptr, DeviceMatrix<float> *dL_dinput = nullptr, bool use_inference_params = false,
                       GradientMode = GradientMode::Overwrite) override {
        if (input.m() == 0) throw std::invalid_argument("batch_size == 0");
        if (!dL_dinput) return;
        if (use_inference_params) throw std::invalid_argument("Cannot use inference params.");
        const ForwardContext &fwd = dynamic_cast<const ForwardContext &>(ctx); // std::bad_cast if the forward pass kept no derivatives
        if (dL_dinput->m() != input.m() || dL_dinput->n() != this->get_input_width() || dL_doutput.m() != input.m() ||
            dL_doutput.n() != this->get_padded_output_width() || fwd.dy_dx.m() != input.m())
            throw std::invalid_argument("Dimension mismatch frequency encoding backward_impl");
        tnn::abi_check(tnn_frequency_backward(dL_doutput.GetPointer(), tnn::dtype_of<T>::value, this->get_padded_output_width(),
                                              fwd.dy_dx.data(), this->get_input_width(), n_frequencies_, dL_dinput->data(), input.m(),
                                              this->get_queue().abi()));
    }

  private:
    struct ForwardContext : public Context {
        ForwardContext(const size_t batch_size, const size_t output_width, tnn::queue &Q) : dy_dx(batch_size, output_width, Q) {}
        DeviceMatrix<float> dy_dx;
    };

    const uint32_t n_frequencies_;
};
