// Multi-resolution hash grid encoding of the native C++ API. Mirrors the host side of the reference's
// include/encodings/grid_interface.h (GridOffsetTable :24-28, GridEncoding :30-54) and include/encodings/grid.h
// (GridEncodingTemplated: constructor :588-659, forward_impl :661-734, backward_impl :736-830, accessors
// :955-983; configuration parsing :1007-1118). The dimension count, the features per level and the hash are
// run-time fields of a descriptor here instead of template parameters; the kernels behind the C ABI of
// libtnn_hip are specialised on them.
#pragma once

#include "encoding.h"

namespace tinydpcppnn {
namespace encodings {
namespace grid {

static constexpr uint32_t MAX_N_LEVELS = TNN_GRID_MAX_LEVELS;
struct GridOffsetTable {
    uint32_t data[MAX_N_LEVELS + 1] = {};
    uint32_t size = 0;
};

template <typename T> class GridEncoding : public Encoding<T> {
  public:
    GridEncoding(const uint32_t input_width, const uint32_t output_width, const uint32_t padded_output_width, tnn::queue &Q)
        : Encoding<T>(input_width, output_width, padded_output_width, Q) {}
    GridEncoding() = delete;
    virtual ~GridEncoding() {}

    virtual uint32_t n_pos_dims() const = 0;
    virtual uint32_t n_features_per_level() const = 0;
    virtual size_t level_n_params(uint32_t level) const = 0;
    virtual size_t level_params_offset(uint32_t level) const = 0;
    virtual const GridOffsetTable &grid_offset_table() const = 0;

    float max_level() const { return m_max_level; }
    void set_max_level(float value) { m_max_level = value; }

  protected:
    float m_max_level = 1000.f; // levels finer than this are skipped; the default disables the feature
};

// One class for every (dimension, features per level, hash) combination the reference instantiates.
template <typename T> class GridEncodingTemplated : public GridEncoding<T> {
  public:
    using grad_t = float;

    GridEncodingTemplated(const uint32_t n_pos_dims, const uint32_t n_features_per_level, const HashType hash_type,
                          const uint32_t padded_output_width, const uint32_t n_features, const uint32_t log2_hashmap_size,
                          const uint32_t base_resolution, const float per_level_scale, const bool stochastic_interpolation,
                          const InterpolationType interpolation_type, const GridType grid_type, tnn::queue &Q)
        : GridEncoding<T>(n_pos_dims, n_features, padded_output_width, Q), m_n_features{n_features},
          m_n_features_per_level{n_features_per_level}, m_stochastic_interpolation{stochastic_interpolation} {
        static_assert(std::is_same<T, float>::value, "the grid encoding of this interface stores float parameters");
        if (n_pos_dims != 2 && n_pos_dims != 3) throw std::runtime_error{"GridEncoding: number of input dims must be 2 or 3."};
        if (n_features_per_level != 1 && n_features_per_level != 2 && n_features_per_level != 4 && n_features_per_level != 8)
            throw std::runtime_error{"GridEncoding: n_features_per_level must be 1, 2, 4, or 8."};
        if (stochastic_interpolation) throw std::invalid_argument("GridEncoding: stochastic interpolation is not supported.");
        const uint32_t n_levels = tinydpcppnn::math::div_round_up(n_features, n_features_per_level);
        if (n_levels > MAX_N_LEVELS)
            throw std::runtime_error("GridEncoding: m_n_levels= " + std::to_string(n_levels) +
                                     " must be at most MAX_N_LEVELS= " + std::to_string(MAX_N_LEVELS));
        if (n_features % n_features_per_level != 0)
            throw std::runtime_error("GridEncoding: n_features= " + std::to_string(n_features) +
                                     " must be a multiple of N_FEATURES_PER_LEVEL = {} " + std::to_string(n_features_per_level));
        tnn::abi_check(tnn_grid_desc_init(&m_desc, n_pos_dims, n_levels, n_features_per_level, log2_hashmap_size, base_resolution,
                                          per_level_scale, (uint32_t)grid_type, (uint32_t)hash_type, (uint32_t)interpolation_type, TNN_FP32));
        for (uint32_t i = 0; i <= n_levels; ++i) m_offset_table.data[i] = m_desc.offsets[i];
        m_offset_table.size = n_levels + 1;

        this->m_params = std::make_shared<DeviceMatrix<T>>(tnn_grid_n_params(&m_desc), 1, this->get_queue());
        this->m_params->fill_random(-1e-4f, 1e-4f).wait();
    }

    std::unique_ptr<Context> forward_impl(const DeviceMatrixView<float> input, DeviceMatrixView<T> *output = nullptr,
                                          bool use_inference_params = false, bool prepare_input_gradients = false) override {
        if (this->get_padded_output_width() == 0) throw std::invalid_argument("Can't have width == 0");
        if (use_inference_params) throw std::invalid_argument("Can't use inference params.");
        if (prepare_input_gradients) throw std::invalid_argument("Can't prepare input gradients");
        if (!output) return nullptr;
        if (output->n() != this->get_padded_output_width()) throw std::invalid_argument("Dimension mismatch grid encoding forw_impl output");
        if (input.n() != this->get_input_width()) throw std::invalid_argument("Dimension mismatch grid encoding forw_impl input");
        if (input.stride() != input.n() || output->stride() != output->n()) throw std::invalid_argument("Only dense matrices are supported.");
        check_max_level();
        const size_t batch = input.m();
        if (batch >= kCellOrderMinBatch) {
            // large batches: order the points by cell first, so that neighbouring lanes gather from the same lines of the
            // table (same rows, bit for bit; the buffer only grows)
            const size_t bytes = tnn_grid_order_bytes(&m_desc, batch);
            if (!m_order || m_order->size() * sizeof(float) < bytes)
                m_order = std::make_unique<DeviceMatrix<float>>((bytes + sizeof(float) - 1) / sizeof(float), 1, this->get_queue());
            tnn::abi_check(tnn_grid_order_points(&m_desc, input.GetPointer(), batch, m_order->data(), m_order->size() * sizeof(float),
                                                 this->get_queue().abi()));
            tnn::abi_check(tnn_grid_forward_ordered(&m_desc, m_order->data(), this->get_params()->data(), output->GetPointer(), TNN_FP32,
                                                    this->get_padded_output_width(), batch, this->get_queue().abi()));
            return nullptr;
        }
        tnn::abi_check(tnn_grid_forward(&m_desc, input.GetPointer(), this->get_params()->data(), output->GetPointer(), TNN_FP32,
                                        this->get_padded_output_width(), batch, this->get_queue().abi()));
        return nullptr; // enqueued on the encoding's in-order stream; the caller waits on the queue when it needs the host to see it
    }

    void backward_impl(const Context &, const DeviceMatrixView<float> input, const DeviceMatrixView<T> dL_doutput,
                       DeviceMatrixView<T> *gradients, DeviceMatrix<float> *dL_dinput = nullptr, bool use_inference_params = false,
                       GradientMode param_gradients_mode = GradientMode::Overwrite) override {
        const size_t batch_size = input.m();
        if (batch_size == 0) throw std::invalid_argument("batch_size == 0");
        if (use_inference_params) throw std::invalid_argument("Cannot use inference params.");
        if (dL_dinput) throw std::invalid_argument("GridEncoding: gradients w.r.t. the input are not supported.");
        if (param_gradients_mode == GradientMode::Ignore) return;
        if (!gradients) throw std::invalid_argument("GridEncoding: gradients must not be null.");
        if (gradients->nelements() != this->get_n_params()) throw std::invalid_argument("GridEncoding: gradients have the wrong size.");
        if (input.n() != this->get_input_width() || dL_doutput.n() != this->get_padded_output_width() || dL_doutput.m() != batch_size)
            throw std::invalid_argument("Dimension mismatch grid encoding backward_impl");
        check_max_level();
        if (batch_size >= kCellOrderMinBackwardBatch) {
            // large batches: the scatter over points in cell order sums neighbouring points on chip before it touches the table.
            // The points are ordered here again (a tenth of the scatter's time): nothing says they are the forward pass's.
            const size_t bytes = tnn_grid_order_bytes(&m_desc, batch_size);
            if (!m_order || m_order->size() * sizeof(float) < bytes)
                m_order = std::make_unique<DeviceMatrix<float>>((bytes + sizeof(float) - 1) / sizeof(float), 1, this->get_queue());
            tnn::abi_check(tnn_grid_order_points(&m_desc, input.GetPointer(), batch_size, m_order->data(), m_order->size() * sizeof(float),
                                                 this->get_queue().abi()));
            tnn::abi_check(tnn_grid_backward_ordered(&m_desc, m_order->data(), dL_doutput.GetPointer(), TNN_FP32, this->get_padded_output_width(),
                                                     gradients->GetPointer(), param_gradients_mode == GradientMode::Overwrite ? 1 : 0,
                                                     batch_size, this->get_queue().abi()));
            return;
        }
        tnn::abi_check(tnn_grid_backward(&m_desc, input.GetPointer(), dL_doutput.GetPointer(), TNN_FP32, this->get_padded_output_width(),
                                         gradients->GetPointer(), param_gradients_mode == GradientMode::Overwrite ? 1 : 0, batch_size,
                                         this->get_queue().abi()));
    }

    uint32_t n_pos_dims() const override { return m_desc.n_dims; }
    uint32_t n_features_per_level() const override { return m_n_features_per_level; }
    size_t level_n_params(uint32_t level) const override {
        return level_params_offset(level + 1) - level_params_offset(level);
    }
    size_t level_params_offset(uint32_t level) const override {
        if (level >= m_offset_table.size) throw std::runtime_error{"Out of bounds params offset request: requested level " +
                                                                    std::to_string(level) + ", but only " +
                                                                    std::to_string(m_offset_table.size) + " levels available."};
        return (size_t)m_offset_table.data[level] * m_n_features_per_level;
    }
    const GridOffsetTable &grid_offset_table() const override { return m_offset_table; }
    const tnn_grid_desc &descriptor() const { return m_desc; }
    uint32_t n_levels() const { return m_desc.n_levels; }

  private:
    void check_max_level() const {
        if (this->m_max_level < (float)m_desc.n_levels) throw std::invalid_argument("GridEncoding: max_level below the level count is not supported.");
    }

    // below this the ordering costs what it saves (2^18 points: 25 us + 42 us against 76 us in 2-D, 25 + 174 against 224 in 3-D
    // with a table of 2^22 entries per level; 2^17: 22 + 28 against 40 and 22 + 97 against 115)
    static constexpr size_t kCellOrderMinBatch = size_t(1) << 18;
    static constexpr size_t kCellOrderMinBackwardBatch = size_t(1) << 17;

    tnn_grid_desc m_desc;
    std::unique_ptr<DeviceMatrix<float>> m_order; // records of the last large batch in cell order
    uint32_t m_n_features;
    uint32_t m_n_features_per_level;
    GridOffsetTable m_offset_table;
    bool m_stochastic_interpolation;
};

// grid.h:1007-1118 of the reference: defaults and the checks on the configuration keys.
template <typename T>
std::shared_ptr<GridEncoding<T>> create_grid_encoding(const json &encoding, std::optional<uint32_t> padded_output_width, tnn::queue &Q) {
    const HashType hash_type = encoding.value(EncodingParams::HASH, HashType::CoherentPrime);
    if ((int)hash_type < 0 || (int)hash_type > (int)HashType::Rng) throw std::runtime_error{"GridEncoding: invalid hash type."};
    const uint32_t n_features_per_level = encoding.value(EncodingParams::N_FEATURES_PER_LEVEL, 2u);
    if (n_features_per_level != 1 && n_features_per_level != 2 && n_features_per_level != 4 && n_features_per_level != 8)
        throw std::runtime_error{"GridEncoding: n_features_per_level must be 1, 2, 4, or 8."};
    const uint32_t log2_hashmap_size = encoding.value(EncodingParams::LOG2_HASHMAP_SIZE, 19u);
    const uint32_t n_dims_to_encode = encoding.value(EncodingParams::N_DIMS_TO_ENCODE, 2u);

    uint32_t n_features;
    if (encoding.contains(EncodingParams::N_FEATURES)) {
        n_features = encoding[EncodingParams::N_FEATURES];
        if (encoding.contains(EncodingParams::N_LEVELS))
            throw std::runtime_error{"GridEncoding: may not specify n_features and n_levels simultaneously (one determines the other)"};
    } else {
        n_features = n_features_per_level * encoding.value(EncodingParams::N_LEVELS, 16u);
    }
    const uint32_t n_levels = n_features / n_features_per_level;
    const GridType grid_type = encoding.value(EncodingParams::GRID_TYPE, GridType::Hash);
    const uint32_t base_resolution = encoding.value(EncodingParams::BASE_RESOLUTION, 16u);
    const float per_level_scale = encoding.value(
        EncodingParams::PER_LEVEL_SCALE,
        grid_type == GridType::Dense ? std::exp(std::log(256.0f / (float)base_resolution) / (n_levels - 1)) : 2.0f);

    if (n_dims_to_encode != 2 && n_dims_to_encode != 3) throw std::runtime_error{"GridEncoding: number of input dims must be 2 or 3."};
    return std::make_shared<GridEncodingTemplated<T>>(
        n_dims_to_encode, n_features_per_level, hash_type, padded_output_width.has_value() ? padded_output_width.value() : n_features,
        n_features, log2_hashmap_size, base_resolution, per_level_scale, encoding.value(EncodingParams::USE_STOCHASTIC_INTERPOLATION, false),
        encoding.value(EncodingParams::INTERPOLATION_METHOD, InterpolationType::Linear), grid_type, Q);
}

} // namespace grid
} // namespace encodings
} // namespace tinydpcppnn
