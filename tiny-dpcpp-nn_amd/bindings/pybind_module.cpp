// Python extension module `tiny_dpcpp_nn_pybind_module`. Mirrors dpcpp_bindings/tiny_dpcpp_nn/pybind_module.cpp
// of the reference: the Activation enum (:150-160), the Module class with its methods (:162-174), create_network
// (:86-138,175-179) and create_encoding (:140-147,180). The modules it hands out run the HIP kernels of
// libtnn_hip through the host classes in include/tnn.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <torch/extension.h>

#include "tnn/tnn_api.h"

namespace py = pybind11;

namespace {

// Python object (dict / list / str / bool / int / float / None) -> configuration value
json to_json(const py::handle &h) {
    if (h.is_none()) return json();
    if (py::isinstance<py::bool_>(h)) return json(h.cast<bool>());
    if (py::isinstance<py::int_>(h)) return json(h.cast<int64_t>());
    if (py::isinstance<py::float_>(h)) return json(h.cast<double>());
    if (py::isinstance<py::str>(h)) return json(h.cast<std::string>());
    if (py::isinstance<py::dict>(h)) {
        json j = json::object();
        for (const auto &kv : py::reinterpret_borrow<py::dict>(h)) j[py::str(kv.first).cast<std::string>()] = to_json(kv.second);
        return j;
    }
    if (py::isinstance<py::list>(h) || py::isinstance<py::tuple>(h)) {
        json j = json::array();
        for (const auto &v : h) j.push_back(to_json(v));
        return j;
    }
    throw std::invalid_argument("encoding config: unsupported value of type " + py::str(py::type::of(h)).cast<std::string>());
}

class PybindingModule {
  public:
    PybindingModule(tnn::Module *module) : m_module{std::unique_ptr<tnn::Module>(module)} {}

    torch::Tensor fwd(torch::Tensor input) {
        CHECK_INPUT(input);
        return m_module->forward_pass(input);
    }
    torch::Tensor inference(torch::Tensor input) {
        CHECK_INPUT(input);
        return m_module->inference(input);
    }
    std::tuple<torch::Tensor, torch::Tensor> bwd_no_encoding_grad(torch::Tensor grad_output, bool pack_gradient, bool get_dl_dinput) {
        CHECK_INPUT(grad_output);
        return m_module->backward_pass(grad_output, pack_gradient, get_dl_dinput);
    }
    std::tuple<torch::Tensor, torch::Tensor> bwd_with_encoding_grad(torch::Tensor grad_output, torch::Tensor input_from_fwd, bool pack_gradient,
                                                                    bool get_dl_dinput) {
        CHECK_INPUT(grad_output);
        return m_module->backward_pass(grad_output, input_from_fwd, pack_gradient, get_dl_dinput);
    }
    /// Network modules: whether inference on `encoding`'s output can run as one kernel, and that inference.
    bool can_fuse_encoding(const PybindingModule &encoding) const { return m_module->can_fuse_encoding(*encoding.m_module); }
    torch::Tensor inference_with_encoding(const PybindingModule &encoding, torch::Tensor positions, bool a_backward_pass_follows) {
        CHECK_INPUT(positions);
        return m_module->inference_with_encoding(*encoding.m_module, positions, a_backward_pass_follows);
    }
    /// Network modules, training without stored activations: inference() is the forward pass, these are the backward passes.
    bool can_recompute_backward() const { return m_module->can_recompute_backward(); }
    std::tuple<torch::Tensor, torch::Tensor> bwd_recompute(torch::Tensor grad_output, torch::Tensor input_from_fwd, bool pack_gradient, bool get_dl_dinput) {
        CHECK_INPUT(grad_output);
        CHECK_INPUT(input_from_fwd);
        return m_module->backward_pass_recompute(grad_output, input_from_fwd, pack_gradient, get_dl_dinput);
    }
    bool can_train_with_encoding(const PybindingModule &encoding) const { return m_module->can_train_with_encoding(*encoding.m_module); }
    std::tuple<torch::Tensor, torch::Tensor> bwd_with_encoding(const PybindingModule &encoding, torch::Tensor positions, torch::Tensor grad_output,
                                                               bool pack_gradient, bool positions_unchanged_since_forward) {
        CHECK_INPUT(positions);
        CHECK_INPUT(grad_output);
        return m_module->backward_with_encoding(*encoding.m_module, positions, grad_output, pack_gradient, positions_unchanged_since_forward);
    }
    torch::Tensor initial_params() { return m_module->initialize_params(); }
    torch::Tensor initial_params(torch::Tensor &tensor) { return m_module->initialize_params(tensor); }
    /// weights_are_packed: the tensor already is in the packed parameter layout, no packing is done
    void set_params(torch::Tensor &tensor, bool weights_are_packed) { m_module->set_params(tensor, weights_are_packed); }
    torch::Tensor get_params() { return m_module->get_params(); }
    uint32_t n_params() const { return (uint32_t)m_module->n_params(); }
    uint32_t n_output_dims() const { return (uint32_t)m_module->n_output_dims(); }

  private:
    std::unique_ptr<tnn::Module> m_module;
};

template <typename T>
PybindingModule create_network_of(int input_width, int output_width, int n_hidden_layers, Activation activation, Activation output_activation,
                                  int width, bool use_bias) {
    switch (width) {
    case 16: return PybindingModule{new tnn::NetworkModule<T, 16>(input_width, output_width, n_hidden_layers, activation, output_activation, use_bias)};
    case 32: return PybindingModule{new tnn::NetworkModule<T, 32>(input_width, output_width, n_hidden_layers, activation, output_activation, use_bias)};
    case 64: return PybindingModule{new tnn::NetworkModule<T, 64>(input_width, output_width, n_hidden_layers, activation, output_activation, use_bias)};
    case 128: return PybindingModule{new tnn::NetworkModule<T, 128>(input_width, output_width, n_hidden_layers, activation, output_activation, use_bias)};
    default: throw std::runtime_error("Unsupported width.");
    }
}

PybindingModule create_network_factory(int input_width, int output_width, int n_hidden_layers, Activation activation,
                                       Activation output_activation, int width, std::string dtype, bool use_bias) {
    if (dtype == "torch.float16")
        return create_network_of<tnn::half>(input_width, output_width, n_hidden_layers, activation, output_activation, width, use_bias);
    if (dtype == "torch.bfloat16")
        return create_network_of<tnn::bf16>(input_width, output_width, n_hidden_layers, activation, output_activation, width, use_bias);
    throw std::runtime_error("Unsupported dtype: " + dtype + ". Only fp16 and bf16 are supported");
}

PybindingModule create_encoding_module(std::string, const py::dict &encoding_config, std::optional<uint32_t> padded_output_width) {
    return PybindingModule{new tnn::EncodingModule<float>(to_json(encoding_config), padded_output_width)};
}

} // namespace

PYBIND11_MODULE(tiny_dpcpp_nn_pybind_module, m) {
    py::enum_<Activation>(m, "Activation")
        .value("ReLU", Activation::ReLU)
        .value("LeakyReLU", Activation::LeakyReLU)
        .value("Exponential", Activation::Exponential)
        .value("Sine", Activation::Sine)
        .value("Sigmoid", Activation::Sigmoid)
        .value("Squareplus", Activation::Squareplus)
        .value("Softplus", Activation::Softplus)
        .value("Tanh", Activation::Tanh)
        .value("Linear", Activation::None)
        .export_values();

    py::class_<PybindingModule>(m, "Module")
        .def("fwd", &PybindingModule::fwd)
        .def("inference", &PybindingModule::inference)
        .def("can_fuse_encoding", &PybindingModule::can_fuse_encoding)
        .def("inference_with_encoding", &PybindingModule::inference_with_encoding, py::arg("encoding"), py::arg("positions"),
             py::arg("a_backward_pass_follows") = false)
        .def("can_recompute_backward", &PybindingModule::can_recompute_backward)
        .def("bwd_recompute", &PybindingModule::bwd_recompute)
        .def("can_train_with_encoding", &PybindingModule::can_train_with_encoding)
        .def("bwd_with_encoding", &PybindingModule::bwd_with_encoding, py::arg("encoding"), py::arg("positions"), py::arg("grad_output"),
             py::arg("pack_gradient"), py::arg("positions_unchanged_since_forward") = false)
        .def("bwd_no_encoding_grad", &PybindingModule::bwd_no_encoding_grad)
        .def("bwd_with_encoding_grad", &PybindingModule::bwd_with_encoding_grad)
        .def("initial_params", py::overload_cast<>(&PybindingModule::initial_params))
        .def("initial_params", py::overload_cast<torch::Tensor &>(&PybindingModule::initial_params))
        .def("set_params", &PybindingModule::set_params)
        .def("get_params", &PybindingModule::get_params)
        .def("n_output_dims", &PybindingModule::n_output_dims)
        .def("n_params", &PybindingModule::n_params);
    m.def("set_initial_weight_seed", [](uint64_t seed) { tnn::set_initial_weight_seed(seed); }, py::arg("seed"),
          "Networks created from now on draw their initial weights from seeds counted up from this one (default: std::random_device, as the reference)");
    m.def("create_network", &create_network_factory, py::arg("input_width"), py::arg("output_width"), py::arg("n_hidden_layers"),
          py::arg("activation"), py::arg("output_activation"), py::arg("width"), py::arg("dtype"), py::arg("use_bias"));
    m.def("create_encoding", &create_encoding_module, py::arg("name"), py::arg("config"), py::arg("padded_output_width") = py::none());
}
