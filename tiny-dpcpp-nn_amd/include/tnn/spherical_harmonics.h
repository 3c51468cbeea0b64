// Spherical-harmonics encoding of 3-D directions given in [0, 1]^3, padded with ones. Mirrors
// include/encodings/spherical_harmonics.h:25-86 of the reference (its backward_impl is not implemented either).
#pragma once

#include "encoding.h"

template <typename T> class SphericalHarmonicsEncoding : public Encoding<T> {
  public:
    SphericalHarmonicsEncoding(const uint32_t degree, const uint32_t n_dims_to_encode, const uint32_t padded_output_width, tnn::queue &Q)
        : Encoding<T>(n_dims_to_encode, degree * degree, padded_output_width, Q), m_degree{degree} {
        if (this->get_input_width() != 3) throw std::runtime_error{"Can only encode 3D directions in spherical harmonics."};
        if (m_degree == 0 || m_degree > 8) throw std::runtime_error{"Spherical harmonics degree > 0 and <= 8."};
    }

    std::unique_ptr<Context> forward_impl(const DeviceMatrixView<float> input, DeviceMatrixView<T> *output = nullptr,
                                          bool use_inference_params = false, bool = false) override {
        if (!output || this->get_padded_output_width() == 0) return std::make_unique<Context>();
        if (input.n() != this->get_input_width()) throw std::invalid_argument("input dimensions do not coincide with encoder");
        if (use_inference_params) throw std::invalid_argument("Cannot yet use inference params");
        if (output->m() != input.m()) throw std::invalid_argument("Differing row numbers");
        if (output->n() != this->get_padded_output_width()) throw std::invalid_argument("number of cols has to be padded output width.");
        if (input.stride() != input.n() || output->stride() != output->n()) throw std::invalid_argument("Only dense matrices are supported.");
        tnn::abi_check(tnn_sh_forward(input.GetPointer(), m_degree, output->GetPointer(), tnn::dtype_of<T>::value,
                                      this->get_padded_output_width(), input.m(), this->get_queue().abi()));
        return std::make_unique<Context>();
    }

    void backward_impl(const Context &, const DeviceMatrixView<float>, const DeviceMatrixView<T>, DeviceMatrixView<T> * = nullptr,
                       DeviceMatrix<float> * = nullptr, bool = false, GradientMode = GradientMode::Overwrite) override {
        throw std::logic_error("Spherical backward not yet implemented.");
    }

  private:
    const uint32_t m_degree;
};
