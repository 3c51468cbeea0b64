// Mirrors include/trainer.h:19-46 of the reference: one training step = forward pass that keeps the
// activations, then the backward pass that produces the weight gradients (no loss, no optimizer; the
// caller supplies dL/d(output) in `losses`). The reference records the step into a SYCL graph when built
// with TEST_GRAPH; here that is a constructor argument. A batch size is run once as enqueued (the network may
// still have to allocate its workspace, which cannot be recorded) and through the graph from then on.
#pragma once

#include "DeviceMatrix.h"
#include "HipGraph.h"
#include "Network.h"

template <typename T> class Trainer {
  public:
    Trainer(Network<T> *network, const bool use_graph = false) : m_network(network), m_use_graph(use_graph) {}

    std::vector<tnn::event> training_step(const DeviceMatrix<T> &input, DeviceMatrices<T> &output, DeviceMatrix<T> &losses,
                                          DeviceMatrices<T> &out_inter_forw, DeviceMatrices<T> &out_inter_backw,
                                          const std::vector<tnn::event> &dependencies) {
        std::vector<tnn::event> deps = {};
        {
            tinydpcppnn::ScopeGuard cg;
            if (m_use_graph && m_warm_rows == input.m()) cg = m_graph.capture_guard(&m_network->get_queue());
            deps = m_network->forward_pass(input, out_inter_forw, dependencies);
            deps = m_network->backward_pass(losses, output, out_inter_backw, out_inter_forw, deps);
        }
        m_warm_rows = input.m();
        return deps;
    }

    const tinydpcppnn::HipGraph &graph() const { return m_graph; }

  private:
    Network<T> *m_network;
    bool m_use_graph;
    size_t m_warm_rows = 0;
    tinydpcppnn::HipGraph m_graph;
};
