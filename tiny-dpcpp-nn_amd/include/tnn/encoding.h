// Encoding base class, configuration keys and enums of the native C++ API. Mirrors
// include/encodings/encoding.h of the reference: EncodingParams (:27-50), EncodingNames (:52-57), the enums
// (:59-88, same ordinals, they cross the C ABI as integers) and Encoding<T> (:90-163).
#pragma once

#include <memory>
#include <optional>

#include "DeviceMatrix.h"
#include "json.h"

struct EncodingParams {
    inline static const std::string ENCODING = "otype";
    inline static const std::string N_DIMS_TO_ENCODE = "n_dims_to_encode";
    inline static const std::string GRID_TYPE = "type";
    inline static const std::string N_LEVELS = "n_levels";
    inline static const std::string N_FEATURES = "n_features";
    inline static const std::string N_FEATURES_PER_LEVEL = "n_features_per_level";
    inline static const std::string LOG2_HASHMAP_SIZE = "log2_hashmap_size";
    inline static const std::string BASE_RESOLUTION = "base_resolution";
    inline static const std::string PER_LEVEL_SCALE = "per_level_scale";
    inline static const std::string DEGREE = "degree";
    inline static const std::string SCALE = "scale";
    inline static const std::string OFFSET = "offset";
    inline static const std::string HASH = "hash";
    inline static const std::string INTERPOLATION_METHOD = "interpolation";
    inline static const std::string USE_STOCHASTIC_INTERPOLATION = "stochastic_interpolation";
    inline static const std::string N_FREQUENCIES = "n_frequencies";
};

struct EncodingNames {
    inline static const std::string IDENTITY = "Identity";
    inline static const std::string SPHERICALHARMONICS = "SphericalHarmonics";
    inline static const std::string GRID = "HashGrid";
    inline static const std::string FREQUENCY = "Frequency";
};

enum class GradientMode { Ignore, Overwrite, Accumulate };
enum class GridType { Hash, Dense, Tiled };
enum class HashType { Prime, CoherentPrime, ReversedPrime, Rng };
enum class InterpolationType { Nearest, Linear, Smoothstep };
enum class ReductionType { Concatenation, Sum, Product };

template <typename T> class Encoding {
  public:
    Encoding() = delete;
    Encoding(const uint32_t input_width, const uint32_t output_width, const uint32_t padded_output_width, tnn::queue &Q)
        : m_params(nullptr), m_input_width(input_width), m_output_width(output_width), m_padded_output_width(padded_output_width), m_q(Q) {
        if (m_input_width == 0) throw std::invalid_argument("Input width cannot be zero");
        if (m_output_width == 0) throw std::invalid_argument("Output width cannot be zero");
        if (m_padded_output_width < m_output_width) throw std::invalid_argument("Padded output width cannot be less than output width");
    }
    virtual ~Encoding() {}

    virtual std::unique_ptr<Context> forward_impl(const DeviceMatrixView<float> input, DeviceMatrixView<T> *output = nullptr,
                                                  bool use_inference_params = false, bool prepare_input_gradients = false) = 0;

    virtual void backward_impl(const Context &ctx, const DeviceMatrixView<float> input, const DeviceMatrixView<T> dL_doutput,
                               DeviceMatrixView<T> *gradients = nullptr, DeviceMatrix<float> *dL_dinput = nullptr,
                               bool use_inference_params = false, GradientMode param_gradients_mode = GradientMode::Overwrite) = 0;

    /// The parameters of the encoding (null for encodings without any). Owned by the encoding.
    std::shared_ptr<DeviceMatrix<T>> get_params() const { return m_params; }
    /// The encoding reads (and its owner trains) its parameters where `params` lies from now on; same number of elements.
    void adopt_params(std::shared_ptr<DeviceMatrix<T>> params) {
        if (!m_params || !params || params->size() != m_params->size()) throw std::invalid_argument("adopt_params: wrong number of parameters");
        m_params = std::move(params);
    }
    uint32_t get_input_width() const { return m_input_width; }
    uint32_t get_padded_output_width() const { return m_padded_output_width; }
    uint32_t get_output_width() const { return m_output_width; }
    uint32_t get_n_to_pad() const { return m_padded_output_width - m_output_width; }
    size_t get_n_params() const { return m_params ? m_params->size() : 0; }
    tnn::queue &get_queue() { return m_q; }

  protected:
    std::shared_ptr<DeviceMatrix<T>> m_params;
    const uint32_t m_input_width;
    const uint32_t m_output_width;
    const uint32_t m_padded_output_width;
    tnn::queue &m_q;
};
