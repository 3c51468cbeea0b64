// Loss base class and the L2 loss of the native C++ API. Mirrors include/losses/loss.h:17-42 and
// include/losses/l2.h:19-40 of the reference: value_i = (p_i - t_i)^2 / N, gradient_i = T(loss_scale * 2 (p_i - t_i) / N).
#pragma once

#include "DeviceMatrix.h"

template <typename T> class Loss {
  public:
    virtual ~Loss() {}

    tnn::event evaluate(tnn::queue &q, const float loss_scale, const DeviceMatrixView<T> &predictions, const DeviceMatrix<float> &targets,
                        DeviceMatrix<float> &values, DeviceMatrix<T> &gradients) {
        SanityCheck(loss_scale, predictions, targets, values, gradients);
        return Kernel(q, predictions.m() * predictions.n(), loss_scale, predictions.GetPointer(), targets.data(), values.data(),
                      gradients.data());
    }

  protected:
    // The reference asserts these; here they throw, so that release builds check them too.
    void SanityCheck(const float loss_scale, const DeviceMatrixView<T> &predictions, const DeviceMatrix<float> &targets,
                     DeviceMatrix<float> &values, DeviceMatrix<T> &gradients) {
        const size_t n_elements = predictions.m() * predictions.n();
        if (predictions.stride() != predictions.n()) throw std::invalid_argument("predictions must be dense");
        if (values.size() != n_elements) throw std::invalid_argument("values size does not match predictions");
        if (gradients.size() != n_elements) throw std::invalid_argument("gradients size does not match predictions");
        if (loss_scale == 0.0f) throw std::invalid_argument("loss_scale must not be 0");
        if (targets.size() != n_elements) throw std::invalid_argument("targets size does not match predictions");
    }

    virtual tnn::event Kernel(tnn::queue &q, const size_t n_elements, const float loss_scale, T const *const predictions,
                              float const *const targets, float *const values, T *const gradients) = 0;
};

template <typename T> class L2Loss : public Loss<T> {
  protected:
    tnn::event Kernel(tnn::queue &q, const size_t n_elements, const float loss_scale, T const *const predictions, float const *const targets,
                      float *const values, T *const gradients) override {
        tnn::abi_check(tnn_l2_loss(tnn::dtype_of<T>::value, predictions, targets, n_elements, loss_scale, values, gradients, q.abi()));
        return tnn::event(q.get());
    }
};
