// Tests of the native C++ host API (tiny-dpcpp-nn_amd/include/tnn) in the manner of the reference's doctests
// (test/doctests/doctest_swiftnet.cpp, doctest_packing.cpp, doctest_losses.cpp, doctest_encodings.cpp,
// doctest_devicematrix.cpp). `--cpu` runs only the cases that need no GPU. The CPU oracle (oracle/tnn_oracle.c) is the
// checker for device results.
#include <cstdio>
#include <functional>
#include <random>

#include "tnn/SwiftNetMLP.h"
#include "tnn/encoding_factory.h"
#include "tnn/io.h"
#include "tnn/loss.h"
#include "tnn/trainer.h"

extern "C" {
void tnn_oracle_round(const float *in, float *out, size_t n, int dtype);
unsigned tnn_oracle_to_packed_layout_coord(unsigned idx, unsigned rows, unsigned cols);
unsigned tnn_oracle_from_packed_layout_coord(unsigned idx, unsigned rows, unsigned cols);
void tnn_oracle_mlp_forward_T(int dtype, int W, int n_mats, int act, int out_act, const float *w, const float *x, size_t M, float *interm,
                              int store_interm);
void tnn_oracle_mlp_backward_T(int dtype, int W, int n_mats, int act, int out_act, const float *w, const float *interm_fwd,
                               const float *dLdy, size_t M, float *interm_bwd, float *dW, float *dX, int round_dw);
void tnn_oracle_l2_loss(int dtype, const float *pred, const float *target, size_t n_elements, float loss_scale, float *values, float *grads);
int tnn_oracle_grid_forward(int n_dims, int n_levels, int F, int log2_hashmap_size, int base_resolution, float per_level_scale,
                            int grid_type, int hash_type, int interp, const float *table, const float *x, size_t M, float *out,
                            int padded_width);
void tnn_oracle_identity_forward(const float *x, int n_dims, float scale, float offset, size_t M, float *out, int padded_width);
void tnn_oracle_frequency_forward(const float *x, int n_dims, int n_freq, size_t M, float *out, int padded_width, float *dy_dx);
void tnn_oracle_frequency_backward(const float *dLdy, int padded_width, const float *dy_dx, int n_dims, int n_freq, size_t M, float *dLdx);
int tnn_oracle_sh_forward(int degree, const float *xin, size_t M, float *out, int padded_width);
int tnn_oracle_grid_backward(int n_dims, int n_levels, int F, int log2_hashmap_size, int base_resolution, float per_level_scale,
                             int grid_type, int hash_type, int interp, const float *x, const float *dLdy, size_t M, int padded_width,
                             float *grad_table);
}

static int g_failed = 0, g_checks = 0;
#define CHECK(cond)                                                                                                                        \
    do {                                                                                                                                   \
        ++g_checks;                                                                                                                        \
        if (!(cond)) {                                                                                                                     \
            ++g_failed;                                                                                                                    \
            std::printf("  CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond);                                                          \
        }                                                                                                                                  \
    } while (0)

template <typename E, typename F> static bool throws(F &&f, const char *needle = nullptr) {
    try {
        f();
    } catch (const E &e) {
        if (needle && std::string(e.what()).find(needle) == std::string::npos) {
            std::printf("  exception text '%s' lacks '%s'\n", e.what(), needle);
            return false;
        }
        return true;
    } catch (const std::exception &e) {
        std::printf("  wrong exception type: %s\n", e.what());
        return false;
    }
    return false;
}

// The reference's metric (include/common/result_check.h:83-102): max-norm difference over the larger max-norm.
static double max_norm_rel(const std::vector<float> &a, const std::vector<float> &b) {
    double d = 0, na = 0, nb = 0;
    for (size_t i = 0; i < a.size(); ++i) {
        d = std::max(d, (double)std::fabs(a[i] - b[i]));
        na = std::max(na, (double)std::fabs(a[i]));
        nb = std::max(nb, (double)std::fabs(b[i]));
    }
    const double n = std::max(na, nb);
    return n == 0 ? d : d / n;
}

template <typename T> static std::vector<float> to_float(const std::vector<T> &v) {
    std::vector<float> f(v.size());
    for (size_t i = 0; i < v.size(); ++i) f[i] = (float)v[i];
    return f;
}
template <typename T> static std::vector<T> from_float(const std::vector<float> &v) {
    std::vector<T> f(v.size());
    for (size_t i = 0; i < v.size(); ++i) f[i] = T(v[i]);
    return f;
}

static std::vector<float> uniform(size_t n, float lo, float hi, uint64_t seed) {
    std::mt19937_64 gen(seed);
    std::uniform_real_distribution<float> dis(lo, hi);
    std::vector<float> v(n);
    for (auto &x : v) x = dis(gen);
    return v;
}

// ------------------------------------------------------------------------------------------- CPU-only cases

static void test_storage_types() {
    // every bf16 pattern round-trips; conversions agree with the oracle's rounding on a spread of floats
    std::vector<float> in;
    for (int e = -30; e <= 20; ++e)
        for (int k = 0; k < 64; ++k) in.push_back(std::ldexp(1.0f + k * 0.0153f + 1e-4f * k, e) * ((k & 1) ? -1.f : 1.f));
    in.push_back(0.f);
    in.push_back(65504.f);
    in.push_back(65520.f);
    in.push_back(1e-8f);
    in.push_back(5.96e-8f);
    in.push_back(2.98e-8f);
    in.push_back(2.9802325e-8f);
    std::vector<float> ob(in.size()), oh(in.size());
    tnn_oracle_round(in.data(), ob.data(), in.size(), TNN_BF16);
    tnn_oracle_round(in.data(), oh.data(), in.size(), TNN_FP16);
    size_t bad = 0;
    for (size_t i = 0; i < in.size(); ++i) {
        if ((float)tnn::bf16(in[i]) != ob[i]) ++bad;
        if ((float)tnn::half(in[i]) != oh[i] && !(std::isinf(oh[i]) && std::isinf((float)tnn::half(in[i])))) ++bad;
    }
    CHECK(bad == 0);
    for (uint32_t b = 0; b < 65536; ++b) {
        tnn::half h;
        h.bits = (uint16_t)b;
        const float f = h;
        if (std::isnan(f)) continue;
        if (tnn::half(f).bits != b) ++bad;
    }
    CHECK(bad == 0);
}

static void test_packed_coords() {
    // doctest_common.cpp:25-119 of the reference pins these point values
    CHECK(toPackedLayoutCoord(0, 4, 4) == 0);
    CHECK(toPackedLayoutCoord(1, 4, 4) == 2);
    CHECK(toPackedLayoutCoord(4, 4, 4) == 1);
    CHECK(toPackedLayoutCoord(5, 4, 4) == 3);
    size_t bad = 0;
    for (unsigned W : {16u, 32u, 64u, 128u})
        for (unsigned i = 0; i < W * W; ++i) {
            if (toPackedLayoutCoord(i, W, W) != tnn_oracle_to_packed_layout_coord(i, W, W)) ++bad;
            if (fromPackedLayoutCoord(i, W, W) != tnn_oracle_from_packed_layout_coord(i, W, W)) ++bad;
            if (fromPackedLayoutCoord(toPackedLayoutCoord(i, W, W), W, W) != i) ++bad;
        }
    CHECK(bad == 0);
    // get_packed_weights: input, hidden and output matrices packed one after the other
    const int W = 16, L = 3;
    std::vector<float> w((L + 1) * W * W);
    for (size_t i = 0; i < w.size(); ++i) w[i] = (float)i;
    const std::vector<float> p = get_packed_weights<float>(w, L, W, W, W);
    for (int m = 0; m <= L; ++m)
        for (int i = 0; i < W * W; ++i)
            if (p[m * W * W + toPackedLayoutCoord(i, W, W)] != w[m * W * W + i]) ++bad;
    CHECK(bad == 0);
    CHECK(throws<std::invalid_argument>([&] { get_packed_weights<float>(std::vector<float>(5), L, W, W, W); }));
}

static void test_json() {
    const json j = json::parse(R"({
        // a comment
        "otype": "HashGrid", "n_levels": 16, /* another */ "per_level_scale": 1.5,
        "stochastic_interpolation": false, "type": "Hash", "list": [1, 2.5, "x"], "nested": {"a": -3}
    })");
    CHECK(j.contains("otype") && !j.contains("missing"));
    CHECK(j["otype"].get<std::string>() == "HashGrid");
    CHECK((uint32_t)j["n_levels"] == 16u);
    CHECK(j.value("per_level_scale", 2.0f) == 1.5f);
    CHECK(j.value("base_resolution", 16u) == 16u);
    CHECK(j.value("stochastic_interpolation", true) == false);
    CHECK(j["list"].size() == 3 && j["list"][1].get<double>() == 2.5 && j["list"][2].is_string());
    CHECK(j["nested"]["a"].get<int>() == -3);
    CHECK(throws<std::out_of_range>([&] { (void)j["missing"]; }));
    CHECK(throws<std::invalid_argument>([&] { json::parse("{\"a\": }"); }));
    CHECK(throws<std::invalid_argument>([&] { json::parse("{\"a\": 1} x"); }));
    const json v = io::validateAndCopyEncodingConfig(j);
    CHECK(v["type"].get<GridType>() == GridType::Hash && j["type"].is_string());
    json bad = j;
    bad["hash"] = "NoSuchHash";
    CHECK(throws<std::runtime_error>([&] { io::validateAndCopyEncodingConfig(bad); }, "Invalid enum value"));
    CHECK(json::parse(j.dump())["n_levels"].get<int>() == 16);
}

// File helpers of io.h: what one writes the other reads back; number files as the reference's own tools write them (one value
// per line) or comma-separated; malformed content and missing files are errors.
static void test_io_files() {
    const std::string dir = "/tmp/tnn_io_test_";
    const std::vector<float> values{0.5f, -1.25f, 3.0f, 1e-3f, 0.1f, -3.4e38f};
    io::saveCSV(dir + "v.csv", values);
    CHECK(io::loadVectorFromCSV<float>(dir + "v.csv") == values); // max_digits10: bit-exact round trip
    CHECK(throws<std::invalid_argument>([&] { io::loadVectorFromCSV<float>(dir + "missing.csv"); }));
    CHECK(throws<std::invalid_argument>([&] { io::saveCSV(std::string("/nonexistent-dir/v.csv"), values); }));
    {
        std::ofstream f(dir + "t.csv");
        f << "1,2;3\r\n4.5, -6\n\n  7e-1\t8";
    }
    CHECK(io::loadVectorFromCSV<float>(dir + "t.csv") == (std::vector<float>{1.f, 2.f, 3.f, 4.5f, -6.f, 0.7f, 8.f}));
    {
        std::ofstream f(dir + "bad.csv");
        f << "1\n2x\n3\n";
    }
    CHECK(throws<std::invalid_argument>([&] { io::loadVectorFromCSV<float>(dir + "bad.csv"); }, "byte 2"));
    {
        std::ofstream f(dir + "huge.csv");
        f << "1e60\n";
    }
    CHECK(throws<std::out_of_range>([&] { io::loadVectorFromCSV<float>(dir + "huge.csv"); }));
    {
        std::ofstream f(dir + "empty.csv");
    }
    CHECK(io::loadVectorFromCSV<float>(dir + "empty.csv").empty());
    {
        std::ofstream f(dir + "cfg.json");
        f << "{\"otype\": \"HashGrid\", \"type\": \"Tiled\", \"interpolation\": \"Smoothstep\", \"n_levels\": 4}";
    }
    const json cfg = io::loadJsonConfig(dir + "cfg.json");
    CHECK(cfg["type"].get<GridType>() == GridType::Tiled && cfg["interpolation"].get<InterpolationType>() == InterpolationType::Smoothstep);
    CHECK(throws<std::runtime_error>([&] { io::loadJsonConfig(dir + "missing.json"); }, "Unable to open"));
    // unpacked [in][out] matrices, one value per line -> the packed parameter vector of a width-16 network
    std::vector<float> w(2 * 16 * 16);
    for (size_t i = 0; i < w.size(); ++i) w[i] = (float)(i % 97) / 128.0f;
    io::saveCSV(dir + "w.csv", w);
    const std::vector<tnn::half> packed = io::load_weights_as_packed_from_file<tnn::half, 16>(dir + "w.csv", 1, 16, 16);
    CHECK(packed.size() == w.size());
    bool same = true;
    for (int m = 0; m < 2; ++m)
        for (int k = 0; k < 16; ++k)
            for (int n = 0; n < 16; ++n) same = same && (float)packed[m * 256 + toPackedLayoutCoord(k * 16 + n, 16, 16)] == w[m * 256 + k * 16 + n];
    CHECK(same);
    CHECK(throws<std::invalid_argument>([&] { (void)io::load_weights_as_packed_from_file<tnn::half, 16>(dir + "w.csv", 2, 16, 16); }, "the network has 768"));
}

// ------------------------------------------------------------------------------------------- GPU cases

template <typename T, int W> static void test_swiftnet(Activation act, Activation out_act, int L, size_t M, int in_w, int out_w, bool use_bias) {
    std::printf(" swiftnet dtype=%d W=%d L=%d act=%d/%d M=%zu in=%d out=%d bias=%d\n", tnn::dtype_of<T>::value, W, L, (int)act, (int)out_act, M,
                in_w, out_w, (int)use_bias);
    std::fflush(stdout);
    const int dtype = tnn::dtype_of<T>::value;
    tnn::queue q;
    SwiftNetMLP<T, W> net(q, in_w, out_w, L, act, out_act, Network<T>::WeightInitMode::xavier_normal, use_bias);
    CHECK(net.get_input_width() == (uint32_t)W && net.get_output_width() == (uint32_t)W);
    CHECK(net.get_unpadded_input_width() == (uint32_t)in_w && net.get_unpadded_output_width() == (uint32_t)out_w);
    CHECK(net.get_n_hidden_layers() == L && net.get_n_hidden_matrices() == L - 1 && net.get_network_width() == W);

    const int n_mats = L + 1;
    const float bound = std::sqrt(6.0f / (2 * W));
    std::vector<float> w_f = uniform((size_t)n_mats * W * W, -bound, bound, 42);
    tnn_oracle_round(w_f.data(), w_f.data(), w_f.size(), dtype);
    net.set_weights_matrices(from_float<T>(w_f), false);

    // what the network holds: packed, with the weights that only see padding zeroed
    const int one_padded = !use_bias ? in_w : (in_w % 16 == 0 ? W : ((in_w + 15) / 16) * 16); // Network.h:194-203 of the reference
    for (int k = 0; k < W; ++k)
        for (int n = 0; n < W; ++n) {
            if (k >= one_padded) w_f[(size_t)k * W + n] = 0.f;
            if (n >= out_w) w_f[((size_t)(n_mats - 1) * W + k) * W + n] = 0.f;
        }
    {
        const std::vector<float> held = to_float(net.get_weights_matrices().copy_to_host());
        const std::vector<float> heldT = to_float(net.get_weightsT_matrices().copy_to_host());
        size_t bad = 0;
        for (int m = 0; m < n_mats; ++m)
            for (int k = 0; k < W; ++k)
                for (int n = 0; n < W; ++n) {
                    const float ref = w_f[((size_t)m * W + k) * W + n];
                    if (held[(size_t)m * W * W + toPackedLayoutCoord(k * W + n, W, W)] != ref) ++bad;
                    if (heldT[(size_t)m * W * W + toPackedLayoutCoord(n * W + k, W, W)] != ref) ++bad;
                }
        CHECK(bad == 0);
    }

    std::vector<float> x_f = uniform(M * W, -1.f, 1.f, 1234);
    for (size_t m = 0; m < M; ++m)
        for (int k = in_w; k < W; ++k) x_f[m * W + k] = (use_bias && k < one_padded) ? 1.f : 0.f;
    tnn_oracle_round(x_f.data(), x_f.data(), x_f.size(), dtype);
    DeviceMatrix<T> x(M, W, q);
    x.copy_from_host(from_float<T>(x_f)).wait();

    // inference
    DeviceMatrix<T> y(M, W, q);
    y.fill(T(123.f)).wait();
    net.inference(x, y, {});
    q.wait();
    std::vector<float> y_ref(M * W);
    tnn_oracle_mlp_forward_T(dtype, W, n_mats, (int)act, (int)out_act, w_f.data(), x_f.data(), M, y_ref.data(), 0);
    const std::vector<float> y_dev = to_float(y.copy_to_host());
    CHECK(max_norm_rel(y_dev, y_ref) <= 1e-2); // the reference's bar (doctest_swiftnet.cpp:183)
    if (out_act != Activation::Sigmoid) {
        size_t bad = 0; // outputs of zeroed weight columns are exactly f_out(0) = 0
        for (size_t m = 0; m < M; ++m)
            for (int n = out_w; n < W; ++n)
                if (y_dev[m * W + n] != 0.f) ++bad;
        CHECK(bad == 0);
    }

    // forward pass that keeps the activations
    DeviceMatrices<T> interm_fwd(L + 2, M, W, M, W, M, W, q);
    net.forward_pass(x, interm_fwd, {});
    q.wait();
    std::vector<float> fwd_ref((size_t)(L + 2) * M * W);
    tnn_oracle_mlp_forward_T(dtype, W, n_mats, (int)act, (int)out_act, w_f.data(), x_f.data(), M, fwd_ref.data(), 1);
    const std::vector<float> fwd_dev = to_float(interm_fwd.copy_to_host());
    CHECK(max_norm_rel(fwd_dev, fwd_ref) <= 1e-2);
    {
        size_t bad = 0;
        for (size_t i = 0; i < M * W; ++i) {
            if (fwd_dev[i] != x_f[i]) ++bad;                                // matrix 0 is the input
            if (fwd_dev[(size_t)(L + 1) * M * W + i] != y_dev[i]) ++bad;    // last matrix equals the inference output
        }
        CHECK(bad == 0);
    }

    // backward pass; the oracle starts from the device's own activations so that only this step is compared
    std::vector<float> g_f = uniform(M * W, -1.f, 1.f, 99);
    for (auto &g : g_f) g *= 1.0f / (float)M;
    tnn_oracle_round(g_f.data(), g_f.data(), g_f.size(), dtype);
    DeviceMatrix<T> g(M, W, q);
    g.copy_from_host(from_float<T>(g_f)).wait();
    DeviceMatrices<T> interm_bwd(L + 1, M, W, M, W, M, W, q);
    DeviceMatrices<T> grads(L + 1, W, W, W, W, W, W, q);
    grads.fill(T(7.f)).wait();
    DeviceMatrix<T> dx(M, W, q);
    DeviceMatrixView<T> dx_view = dx.GetView();
    net.backward_pass(g, grads, interm_bwd, interm_fwd, {}, &dx_view);
    q.wait();
    std::vector<float> bwd_ref((size_t)(L + 1) * M * W), dW_ref((size_t)n_mats * W * W), dX_ref(M * W);
    tnn_oracle_mlp_backward_T(dtype, W, n_mats, (int)act, (int)out_act, w_f.data(), fwd_dev.data(), g_f.data(), M, bwd_ref.data(),
                              dW_ref.data(), dX_ref.data(), 1);
    CHECK(max_norm_rel(to_float(interm_bwd.copy_to_host()), bwd_ref) <= 1e-2);
    const std::vector<float> dW_dev = to_float(grads.copy_to_host());
    CHECK(max_norm_rel(dW_dev, dW_ref) <= 1e-2);
    CHECK(max_norm_rel(to_float(dx.copy_to_host()), dX_ref) <= 1e-2);

    // Trainer::training_step == forward_pass + backward_pass
    {
        Trainer<T> trainer(&net);
        DeviceMatrices<T> f2(L + 2, M, W, M, W, M, W, q), b2(L + 1, M, W, M, W, M, W, q), g2(L + 1, W, W, W, W, W, W, q);
        trainer.training_step(x, g2, g, f2, b2, {});
        q.wait();
        CHECK(to_float(f2.copy_to_host()) == fwd_dev);
        CHECK(max_norm_rel(to_float(g2.copy_to_host()), dW_dev) <= 1e-3); // fp32 partial sums may be added in another order
    }

    // PackAndTranspose (in place, as the reference's module calls it): [out][in] raw -> parameter layout
    {
        grads.PackAndTranspose(grads);
        const std::vector<float> packed = to_float(grads.copy_to_host());
        size_t bad = 0;
        for (int m = 0; m < n_mats; ++m)
            for (int k = 0; k < W; ++k)
                for (int n = 0; n < W; ++n)
                    if (packed[(size_t)m * W * W + toPackedLayoutCoord(k * W + n, W, W)] != dW_dev[((size_t)m * W + n) * W + k]) ++bad;
        CHECK(bad == 0);
    }
}

static void test_swiftnet_constant_weights() {
    // doctest_swiftnet.cpp:44-96 of the reference: weights 0.01, activation None => every output is x * (0.01 W)^(L+1)
    // up to the rounding of each layer.
    std::printf(" swiftnet constant weights\n");
    tnn::queue q;
    const int W = 64, L = 2;
    const size_t M = 64;
    SwiftNetMLP<tnn::bf16, 64> net(q, W, W, L, Activation::None, Activation::None, Network<tnn::bf16>::WeightInitMode::constant_pos);
    DeviceMatrix<tnn::bf16> x(M, W, q), y(M, W, q);
    x.fill(tnn::bf16(0.5f)).wait();
    net.inference(x, y, {});
    q.wait();
    float v = 0.5f;
    const float w = (float)tnn::bf16(0.01f);
    for (int l = 0; l <= L; ++l) v = (float)tnn::bf16(v * w * W);
    const std::vector<float> out = to_float(y.copy_to_host());
    size_t bad = 0;
    for (float o : out)
        if (std::fabs(o - v) > 1e-2f * std::fabs(v)) ++bad;
    CHECK(bad == 0);
}

static void test_swiftnet_errors() {
    std::printf(" swiftnet error paths\n");
    tnn::queue q;
    using bf = tnn::bf16;
    CHECK(throws<std::runtime_error>([&] { SwiftNetMLP<bf, 64> n(q, 65, 64, 2, Activation::ReLU, Activation::None); }, "Input width of 128"));
    CHECK(throws<std::runtime_error>([&] { SwiftNetMLP<bf, 64> n(q, 64, 200, 2, Activation::ReLU, Activation::None); }, "not supported"));
    CHECK(throws<std::invalid_argument>([&] { SwiftNetMLP<bf, 64> n(q, 0, 64, 2, Activation::ReLU, Activation::None); }, "width <= 0 cannot be padded"));
    CHECK(throws<std::runtime_error>([&] { SwiftNetMLP<bf, 64> n(q, 64, 64, 0, Activation::ReLU, Activation::None); }, "must be >= 1"));
    CHECK(throws<std::invalid_argument>([&] { SwiftNetMLP<bf, 64> n(q, 64, 64, -1, Activation::ReLU, Activation::None); }, "non-negative"));
    CHECK(throws<std::runtime_error>([&] { SwiftNetMLP<bf, 64> n(q, 64, 64, 2, Activation::Tanh, Activation::None); }, "m_activation must be"));
    CHECK(throws<std::runtime_error>([&] { SwiftNetMLP<bf, 64> n(q, 64, 64, 2, Activation::ReLU, Activation::Sine); }, "m_output_activation"));
    CHECK(throws<std::invalid_argument>(
        [&] { SwiftNetMLP<bf, 64> n(q, 64, 64, 2, Activation::ReLU, Activation::None, Network<bf>::WeightInitMode::arange); }, "arange"));

    SwiftNetMLP<bf, 64> net(q, 64, 64, 2, Activation::ReLU, Activation::None);
    CHECK(throws<std::runtime_error>([&] { net.set_weights_matrices(std::vector<bf>(10), false); }, "does not match"));
    DeviceMatrix<bf> x7(7, 64, q), y7(7, 64, q), x8(8, 64, q), y8(8, 64, q), x8n(8, 32, q), y16(16, 64, q);
    CHECK(throws<std::invalid_argument>([&] { net.inference(x7, y7, {}); }, "divisible by 8"));
    CHECK(throws<std::invalid_argument>([&] { net.inference(x8n, y8, {}); }, "Input array too small"));
    CHECK(throws<std::invalid_argument>([&] { net.inference(x8, y16, {}); }, "Output array too small"));
    DeviceMatrices<bf> f_ok(4, 8, 64, 8, 64, 8, 64, q), f_few(3, 8, 64, 8, 64, 8, 64, q), f_m(4, 16, 64, 16, 64, 16, 64, q);
    CHECK(throws<std::invalid_argument>([&] { net.forward_pass(x8, f_few, {}); }, "Not enough matrices"));
    CHECK(throws<std::invalid_argument>([&] { net.forward_pass(x8, f_m, {}); }, "doesn't match input shape"));
    CHECK(throws<std::invalid_argument>([&] { net.forward_pass(x7, f_ok, {}); }, "divisible by 8"));
    DeviceMatrices<bf> b_ok(3, 8, 64, 8, 64, 8, 64, q), b_few(2, 8, 64, 8, 64, 8, 64, q), g_ok(3, 64, 64, 64, 64, 64, 64, q),
        g_few(2, 64, 64, 64, 64, 64, 64, q);
    CHECK(throws<std::invalid_argument>([&] { net.backward_pass(x8, g_ok, b_few, f_ok, {}); }, "intermediate_output_backward"));
    CHECK(throws<std::invalid_argument>([&] { net.backward_pass(x8, g_few, b_ok, f_ok, {}); }, "output of backward pass"));
    CHECK(throws<std::invalid_argument>([&] { net.backward_pass(x8, g_ok, b_ok, f_few, {}); }, "intermediate_output_forward"));
    net.forward_pass(x8, f_ok, {});
    net.backward_pass(x8, g_ok, b_ok, f_ok, {});
    q.wait();

    // matrices and views
    CHECK(throws<std::invalid_argument>([&] { x8.GetView(9, 64, 0, 0); }, "OOB"));
    CHECK(throws<std::invalid_argument>([&] { x8.copy_from_host(std::vector<bf>(3)); }));
    CHECK(throws<std::invalid_argument>([&] { f_ok.GetView(4); }, "Invalid idx"));
    CHECK(throws<std::invalid_argument>([&] { x8 = x7; }, "differing dimensions"));
    const DeviceMatrixView<bf> sub = f_ok.GetView(2);
    CHECK(sub.m() == 8 && sub.n() == 64 && sub.GetPointer() == f_ok.data() + 2 * 8 * 64);
    CHECK(f_ok.GetViews().GetElementPointer(3, 1, 2) == f_ok.data() + 3 * 8 * 64 + 64 + 2);
}

// Trainer with graph recording: every step equals the step run as enqueued (SyclGraph use in include/trainer.h:27-31)
static void test_trainer_graph() {
    std::printf(" trainer with HIP graph\n");
    hipStream_t raw = nullptr;
    tnn::hip_check(hipStreamCreate(&raw), "hipStreamCreate");
    {
        tnn::queue q(raw);
        typedef tnn::bf16 T;
        const int W = 64, L = 3;
        const size_t M = 2048;
        SwiftNetMLP<T, 64> net(q, W, W, L, Activation::ReLU, Activation::None);
        Trainer<T> eager(&net, false), recorded(&net, true);
        DeviceMatrix<T> x(M, W, q), g(M, W, q);
        DeviceMatrices<T> f1(L + 2, M, W, M, W, M, W, q), b1(L + 1, M, W, M, W, M, W, q), w1(L + 1, W, W, W, W, W, W, q);
        DeviceMatrices<T> f2(L + 2, M, W, M, W, M, W, q), b2(L + 1, M, W, M, W, M, W, q), w2(L + 1, W, W, W, W, W, W, q);
        for (int it = 0; it < 4; ++it) {
            x.copy_from_host(from_float<T>(uniform(M * W, -1.f, 1.f, 100 + it)));
            g.copy_from_host(from_float<T>(uniform(M * W, -1e-3f, 1e-3f, 200 + it)));
            eager.training_step(x, w1, g, f1, b1, {});
            q.wait();
            f2.fill(T(9.f)).wait();
            w2.fill(T(9.f)).wait();
            recorded.training_step(x, w2, g, f2, b2, {});
            q.wait();
            CHECK(to_float(f1.copy_to_host()) == to_float(f2.copy_to_host()));
            CHECK(to_float(b1.copy_to_host()) == to_float(b2.copy_to_host()));
            CHECK(max_norm_rel(to_float(w1.copy_to_host()), to_float(w2.copy_to_host())) <= 1e-3);
        }
        CHECK(recorded.graph().launches() == 3 && eager.graph().launches() == 0); // the first step of a batch size is not recorded
        // the legacy default stream cannot be recorded: the step then simply runs
        tnn::queue q0;
        tinydpcppnn::HipGraph none;
        { auto guard = none.capture_guard(&q0); }
        { auto guard = none.capture_guard(nullptr); }
        CHECK(none.launches() == 0);
    }
    tnn::hip_check(hipStreamDestroy(raw), "hipStreamDestroy");
}

static void test_l2_loss() {
    std::printf(" l2 loss\n");
    tnn::queue q;
    // doctest_losses.cpp:46-51 of the reference: closed form on constant predictions and targets
    const size_t M = 64, N = 16;
    const float loss_scale = 128.f, p = 0.25f, t = 1.0f;
    DeviceMatrix<tnn::half> pred(M, N, q), grads(M, N, q);
    DeviceMatrix<float> targets(M, N, q), values(M, N, q);
    pred.fill(tnn::half(p)).wait();
    targets.fill(t).wait();
    L2Loss<tnn::half> loss;
    loss.evaluate(q, loss_scale, pred.GetView(), targets, values, grads).wait();
    const std::vector<float> v = values.copy_to_host(), g = to_float(grads.copy_to_host());
    size_t bad = 0;
    const float n = (float)(M * N);
    for (size_t i = 0; i < v.size(); ++i) {
        if (std::fabs(v[i] - (p - t) * (p - t) / n) > 1e-9f) ++bad;
        if (g[i] != (float)tnn::half(loss_scale * 2 * (p - t) / n)) ++bad;
    }
    CHECK(bad == 0);
    // seeded values against the oracle
    std::vector<float> pf = uniform(M * N, -2, 2, 5), tf = uniform(M * N, -2, 2, 6), vr(M * N), gr(M * N);
    tnn_oracle_round(pf.data(), pf.data(), pf.size(), TNN_FP16);
    pred.copy_from_host(from_float<tnn::half>(pf));
    targets.copy_from_host(tf);
    loss.evaluate(q, loss_scale, pred.GetView(), targets, values, grads).wait();
    tnn_oracle_l2_loss(TNN_FP16, pf.data(), tf.data(), M * N, loss_scale, vr.data(), gr.data());
    CHECK(values.copy_to_host() == vr);
    CHECK(to_float(grads.copy_to_host()) == gr);
    DeviceMatrix<float> small(2, 2, q);
    CHECK(throws<std::invalid_argument>([&] { loss.evaluate(q, loss_scale, pred.GetView(), small, values, grads); }));
    CHECK(throws<std::invalid_argument>([&] { loss.evaluate(q, 0.f, pred.GetView(), targets, values, grads); }));
}

static void test_grid(const char *config_text, uint32_t padded_width, size_t M) {
    std::printf(" grid %s\n", config_text);
    std::fflush(stdout);
    tnn::queue q;
    const json config = io::validateAndCopyEncodingConfig(json::parse(config_text));
    std::shared_ptr<Encoding<float>> enc = create_encoding<float>(config, q, padded_width);
    auto *grid = dynamic_cast<tinydpcppnn::encodings::grid::GridEncodingTemplated<float> *>(enc.get());
    CHECK(grid != nullptr);
    const tnn_grid_desc &d = grid->descriptor();
    const uint32_t D = d.n_dims, F = d.n_features_per_level, L = d.n_levels;
    CHECK(enc->get_input_width() == D && enc->get_output_width() == L * F && enc->get_padded_output_width() == padded_width);
    CHECK(enc->get_n_params() == (size_t)d.offsets[L] * F && grid->level_params_offset(1) == (size_t)d.offsets[1] * F);
    CHECK(grid->level_n_params(0) == (size_t)(d.offsets[1] - d.offsets[0]) * F);

    // default initialisation: uniform in +-1e-4
    std::vector<float> table = enc->get_params()->copy_to_host();
    {
        double mean = 0;
        size_t bad = 0;
        for (float v : table) {
            mean += v;
            if (!(v >= -1e-4f && v < 1e-4f)) ++bad;
        }
        CHECK(bad == 0 && std::fabs(mean / table.size()) < 1e-5);
    }
    table = uniform(table.size(), -1.f, 1.f, 7);
    enc->get_params()->copy_from_host(table);

    std::vector<float> x = uniform(M * D, 0.f, 1.f, 11);
    x[0] = 0.f;
    x[D] = 1.f; // the wrap-around corner
    DeviceMatrix<float> xd(M, D, q), out(M, padded_width, q);
    xd.copy_from_host(x);
    out.fill(55.f).wait();
    DeviceMatrixView<float> out_view = out.GetView();
    enc->forward_impl(xd.GetView(), &out_view);
    std::vector<float> ref(M * padded_width);
    CHECK(tnn_oracle_grid_forward(D, L, F, d.log2_hashmap_size, d.base_resolution, d.per_level_scale, d.grid_type, d.hash_type,
                                  d.interpolation, table.data(), x.data(), M, ref.data(), padded_width) == 0);
    const std::vector<float> dev = out.copy_to_host();
    double worst = 0;
    for (size_t i = 0; i < dev.size(); ++i) worst = std::max(worst, (double)std::fabs(dev[i] - ref[i]));
    CHECK(worst <= 2e-6); // fp32 blends of values in [-1, 1]: only the order of a handful of fused operations differs

    std::vector<float> dy = uniform(M * padded_width, -1.f, 1.f, 13);
    DeviceMatrix<float> dyd(M, padded_width, q), grads(enc->get_n_params(), 1, q);
    dyd.copy_from_host(dy);
    grads.fill(3.f).wait();
    DeviceMatrixView<float> grads_view = grads.GetView();
    Context ctx;
    enc->backward_impl(ctx, xd.GetView(), dyd.GetView(), &grads_view);
    q.wait();
    std::vector<float> gref(table.size());
    CHECK(tnn_oracle_grid_backward(D, L, F, d.log2_hashmap_size, d.base_resolution, d.per_level_scale, d.grid_type, d.hash_type,
                                   d.interpolation, x.data(), dy.data(), M, padded_width, gref.data()) == 0);
    const std::vector<float> gdev = grads.copy_to_host();
    CHECK(max_norm_rel(gdev, gref) <= 1e-5);
    // Accumulate adds to what is there; Ignore leaves it alone
    enc->backward_impl(ctx, xd.GetView(), dyd.GetView(), &grads_view, nullptr, false, GradientMode::Accumulate);
    q.wait();
    std::vector<float> twice(gref.size());
    for (size_t i = 0; i < gref.size(); ++i) twice[i] = 2 * gref[i];
    CHECK(max_norm_rel(grads.copy_to_host(), twice) <= 1e-5);
    const std::vector<float> before = grads.copy_to_host();
    enc->backward_impl(ctx, xd.GetView(), dyd.GetView(), &grads_view, nullptr, false, GradientMode::Ignore);
    q.wait();
    CHECK(grads.copy_to_host() == before);

    DeviceMatrix<float> wrong(M, padded_width + 16, q);
    DeviceMatrixView<float> wrong_view = wrong.GetView();
    CHECK(throws<std::invalid_argument>([&] { enc->forward_impl(xd.GetView(), &wrong_view); }, "Dimension mismatch"));
    CHECK(throws<std::invalid_argument>([&] { enc->forward_impl(xd.GetView(), &out_view, true); }, "inference params"));
    CHECK(enc->forward_impl(xd.GetView(), nullptr) == nullptr);
}

static double max_abs_diff(const std::vector<float> &a, const std::vector<float> &b) {
    double d = 0;
    for (size_t i = 0; i < a.size(); ++i) d = std::max(d, (double)std::fabs(a[i] - b[i]));
    return d;
}

// test/doctest_encodings.cpp:156-232,346-584 of the reference, plus the oracle on seeded inputs
static void test_parameter_free_encodings() {
    std::printf(" identity / frequency / spherical harmonics\n");
    tnn::queue q;
    const size_t M = 500;
    std::vector<float> x = uniform(M * 3, 0.f, 1.f, 21);
    DeviceMatrix<float> xd(M, 3, q);
    xd.copy_from_host(x);
    {
        auto enc = create_encoding<float>(json::parse(R"({"otype": "Identity", "n_dims_to_encode": 3, "scale": 1.5, "offset": 0.25})"), q, 8u);
        CHECK(enc->get_input_width() == 3 && enc->get_output_width() == 3 && enc->get_padded_output_width() == 8 && enc->get_n_params() == 0 &&
              enc->get_params() == nullptr && enc->get_n_to_pad() == 5);
        DeviceMatrix<float> out(M, 8, q);
        DeviceMatrixView<float> v = out.GetView();
        CHECK(enc->forward_impl(xd.GetView(), &v) != nullptr);
        std::vector<float> ref(M * 8);
        tnn_oracle_identity_forward(x.data(), 3, 1.5f, 0.25f, M, ref.data(), 8);
        CHECK(out.copy_to_host() == ref);
        Context ctx;
        CHECK(throws<std::logic_error>([&] { enc->backward_impl(ctx, xd.GetView(), v); }, "Not yet implemented"));
        DeviceMatrix<float> bad(M, 9, q);
        DeviceMatrixView<float> bv = bad.GetView();
        CHECK(throws<std::invalid_argument>([&] { enc->forward_impl(xd.GetView(), &bv); }, "padded output width"));
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "Identity", "n_dims_to_encode": 3, "scale": 1.0})"), q); },
                                            "Config misses offset"));
    }
    {
        const json cfg = json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 3, "n_frequencies": 6})");
        auto enc = create_encoding<float>(cfg, q, 48u);
        CHECK(enc->get_output_width() == 36 && enc->get_padded_output_width() == 48);
        CHECK(create_encoding<float>(cfg, q)->get_padded_output_width() == 36);
        DeviceMatrix<float> out(M, 48, q);
        DeviceMatrixView<float> v = out.GetView();
        std::unique_ptr<Context> ctx = enc->forward_impl(xd.GetView(), &v, false, true);
        std::vector<float> ref(M * 48), dy(M * 36);
        tnn_oracle_frequency_forward(x.data(), 3, 6, M, ref.data(), 48, dy.data());
        CHECK(max_abs_diff(out.copy_to_host(), ref) <= 2e-6);
        std::vector<float> g = uniform(M * 48, -1.f, 1.f, 22), dref(M * 3);
        DeviceMatrix<float> gd(M, 48, q), dx(M, 3, q);
        gd.copy_from_host(g);
        enc->backward_impl(*ctx, xd.GetView(), gd.GetView(), nullptr, &dx);
        const std::vector<float> dxh = dx.copy_to_host();
        // the oracle gets its own derivatives; cos of arguments up to 32 pi differs by ulps between host and device
        tnn_oracle_frequency_backward(g.data(), 48, dy.data(), 3, 6, M, dref.data());
        CHECK(max_norm_rel(dxh, dref) <= 1e-4);
        std::unique_ptr<Context> plain = enc->forward_impl(xd.GetView(), &v);
        CHECK(throws<std::bad_cast>([&] { enc->backward_impl(*plain, xd.GetView(), gd.GetView(), nullptr, &dx); }));
        // creation cases of the reference's doctest
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 1})"), q); }));
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 1, "n_frequencies": 0})"), q); }));
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 1, "n_frequencies": -1})"), q); }));
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 0, "n_frequencies": 1})"), q); }));
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 1, "n_frequencies": 1})"), q, 1u); }));
        CHECK(create_encoding<float>(json::parse(R"({"otype": "Frequency", "n_dims_to_encode": 1, "n_frequencies": 1})"), q, 2u) != nullptr);
    }
    {
        auto enc = create_encoding<float>(json::parse(R"({"otype": "SphericalHarmonics", "n_dims_to_encode": 3, "degree": 4})"), q, 32u);
        CHECK(enc->get_output_width() == 16 && enc->get_padded_output_width() == 32);
        DeviceMatrix<float> out(M, 32, q);
        DeviceMatrixView<float> v = out.GetView();
        enc->forward_impl(xd.GetView(), &v);
        q.wait();
        std::vector<float> ref(M * 32);
        CHECK(tnn_oracle_sh_forward(4, x.data(), M, ref.data(), 32) == 0);
        CHECK(max_abs_diff(out.copy_to_host(), ref) <= 2e-5);
        Context ctx;
        CHECK(throws<std::logic_error>([&] { enc->backward_impl(ctx, xd.GetView(), v); }, "not yet implemented"));
        CHECK(throws<std::runtime_error>([&] { create_encoding<float>(json::parse(R"({"otype": "SphericalHarmonics", "n_dims_to_encode": 2, "degree": 4})"), q); },
                                         "3D directions"));
        CHECK(throws<std::runtime_error>([&] { create_encoding<float>(json::parse(R"({"otype": "SphericalHarmonics", "n_dims_to_encode": 3, "degree": 9})"), q); },
                                         "degree"));
        CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse(R"({"otype": "SphericalHarmonics", "n_dims_to_encode": 3})"), q); },
                                            "Config misses degree"));
    }
}

static void test_encoding_config_errors() {
    std::printf(" encoding configuration errors\n");
    tnn::queue q;
    CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse("{\"n_levels\": 4}"), q); }, "otype"));
    CHECK(throws<std::invalid_argument>([&] { create_encoding<float>(json::parse("{\"otype\": \"Nope\"}"), q); }, "Unknown encoding type"));
    CHECK(throws<std::runtime_error>(
        [&] { create_encoding<float>(json::parse("{\"otype\": \"HashGrid\", \"n_levels\": 4, \"n_features\": 8}"), q); }, "simultaneously"));
    CHECK(throws<std::runtime_error>([&] { create_encoding<float>(json::parse("{\"otype\": \"HashGrid\", \"n_dims_to_encode\": 4}"), q); },
                                     "2 or 3"));
    CHECK(throws<std::runtime_error>([&] { create_encoding<float>(json::parse("{\"otype\": \"HashGrid\", \"n_features_per_level\": 3}"), q); },
                                     "1, 2, 4, or 8"));
    CHECK(throws<std::invalid_argument>(
        [&] { create_encoding<float>(json::parse("{\"otype\": \"HashGrid\", \"n_levels\": 4, \"log2_hashmap_size\": 10}"), q, 4u); },
        "Padded output width"));
}

int main(int argc, char **argv) {
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu";
    std::printf("storage types\n");
    test_storage_types();
    std::printf("packed coordinates\n");
    test_packed_coords();
    std::printf("json\n");
    test_json();
    std::printf("io files\n");
    test_io_files();
    if (!cpu_only) {
        tnn::abi_check(tnn_device_check());
        std::printf("swiftnet\n");
        test_swiftnet_constant_weights();
        test_swiftnet_errors();
        test_swiftnet<tnn::bf16, 64>(Activation::ReLU, Activation::None, 4, 1024, 64, 64, false);
        test_swiftnet<tnn::bf16, 64>(Activation::ReLU, Activation::None, 2, 512, 32, 3, false);
        test_swiftnet<tnn::bf16, 64>(Activation::ReLU, Activation::None, 2, 512, 3, 5, true);
        test_swiftnet<tnn::bf16, 64>(Activation::ReLU, Activation::None, 2, 64, 32, 64, true);
        test_swiftnet<tnn::half, 16>(Activation::Sigmoid, Activation::None, 2, 256, 16, 16, false);
        test_swiftnet<tnn::half, 32>(Activation::None, Activation::Sigmoid, 4, 256, 20, 32, true);
        test_swiftnet<tnn::half, 128>(Activation::ReLU, Activation::ReLU, 8, 256, 128, 100, false);
        test_swiftnet<tnn::bf16, 128>(Activation::None, Activation::None, 1, 8, 128, 128, false);
        test_l2_loss();
        test_trainer_graph();
        std::printf("encodings\n");
        test_grid(R"({"otype": "HashGrid", "n_dims_to_encode": 2, "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 15,
                      "base_resolution": 16, "per_level_scale": 1.5})", 32, 2048);
        test_grid(R"({"otype": "HashGrid", "n_dims_to_encode": 3, "n_levels": 8, "n_features_per_level": 2, "log2_hashmap_size": 14,
                      "base_resolution": 4, "per_level_scale": 1.447, "hash": "Prime"})", 64, 1000);
        test_grid(R"({"otype": "HashGrid", "type": "Dense", "n_dims_to_encode": 2, "n_levels": 4, "n_features_per_level": 4,
                      "base_resolution": 8, "interpolation": "Smoothstep"})", 16, 777);
        test_grid(R"({"otype": "HashGrid", "type": "Tiled", "n_dims_to_encode": 3, "n_features": 6, "n_features_per_level": 1,
                      "base_resolution": 5, "per_level_scale": 2.0, "interpolation": "Nearest"})", 16, 256);
        test_parameter_free_encodings();
        test_encoding_config_errors();
    }
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed == 0 ? 0 : 1;
}
