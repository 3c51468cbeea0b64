// Identity encoding: out = in * scale + offset, padded with ones. Mirrors include/encodings/identity.h:26-116 of the
// reference (its backward_impl throws "Not yet implemented." before doing anything; so does this one).
#pragma once

#include "encoding.h"

template <typename T> class IdentityEncoding : public Encoding<T> {
  public:
    IdentityEncoding(const uint32_t n_dims_to_encode, const uint32_t padded_output_width, const float scale, const float offset, tnn::queue &Q)
        : Encoding<T>(n_dims_to_encode, n_dims_to_encode, padded_output_width, Q), m_scale{scale}, m_offset{offset} {}

    std::unique_ptr<Context> forward_impl(const DeviceMatrixView<float> input, DeviceMatrixView<T> *output = nullptr,
                                          bool use_inference_params = false, bool prepare_input_gradients = false) override {
        if (!output || this->get_padded_output_width() == 0) return std::make_unique<Context>();
        if (input.n() != this->get_input_width()) throw std::invalid_argument("input dimensions do not coincide with encoder");
        if (use_inference_params) throw std::invalid_argument("Cannot yet use inference params");
        if (prepare_input_gradients) throw std::invalid_argument("Identity encoding cannot yet prepare input gradients");
        if (output->m() != input.m()) throw std::invalid_argument("Differing row numbers");
        if (output->n() != this->get_padded_output_width()) throw std::invalid_argument("number of cols has to be padded output width.");
        if (input.stride() != input.n() || output->stride() != output->n()) throw std::invalid_argument("Only dense matrices are supported.");
        tnn::abi_check(tnn_identity_forward(input.GetPointer(), this->get_input_width(), m_scale, m_offset, output->GetPointer(),
                                            tnn::dtype_of<T>::value, this->get_padded_output_width(), input.m(), this->get_queue().abi()));
        return std::make_unique<Context>();
    }

    void backward_impl(const Context &, const DeviceMatrixView<float>, const DeviceMatrixView<T>, DeviceMatrixView<T> * = nullptr,
                       DeviceMatrix<float> * = nullptr, bool = false, GradientMode = GradientMode::Overwrite) override {
        throw std::logic_error("Not yet implemented.");
    }

  private:
    const float m_scale;
    const float m_offset;
};
