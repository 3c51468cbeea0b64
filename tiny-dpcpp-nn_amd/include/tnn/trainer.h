// Mirrors include/trainer.h:19-46 of the reference: one training step = forward pass that keeps the
// activations, then the backward pass that produces the weight gradients (no loss, no optimizer; the
// caller supplies dL/d(output) in `losses`).
#pragma once

#include "DeviceMatrix.h"
#include "Network.h"

template <typename T> class Trainer {
  public:
    Trainer(Network<T> *network) : m_network(network) {}

    std::vector<tnn::event> training_step(const DeviceMatrix<T> &input, DeviceMatrices<T> &output, DeviceMatrix<T> &losses,
                                          DeviceMatrices<T> &out_inter_forw, DeviceMatrices<T> &out_inter_backw,
                                          const std::vector<tnn::event> &dependencies) {
        std::vector<tnn::event> deps = m_network->forward_pass(input, out_inter_forw, dependencies);
        return m_network->backward_pass(losses, output, out_inter_backw, out_inter_forw, deps);
    }

  private:
    Network<T> *m_network;
};
