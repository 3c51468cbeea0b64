// create_encoding: configuration -> encoding object, the one boundary function of the reference's
// include/encodings/encoding_factory.h (:112-180). Same configuration keys, defaults, warnings and exception types;
// the construction is a table from the "otype" name to a builder function instead of a factory class per encoding.
#pragma once

#include <array>
#include <iostream>
#include <limits>

#include "encoding.h"
#include "frequency.h"
#include "grid.h"
#include "identity.h"
#include "spherical_harmonics.h"

namespace tnn {
namespace encoding_builders {

template <typename T> using Built = std::shared_ptr<Encoding<T>>;
template <typename T> using Builder = Built<T> (*)(const json &, std::optional<uint32_t>, tnn::queue &);

// A key that the encoding cannot be built without.
inline const json &need(const json &config, const std::string &key) {
    if (!config.contains(key)) throw std::invalid_argument("Config misses " + key);
    return config[key];
}

// A count that must fit 32 bits. The reference reads these as uint32_t and lets a negative number wrap to a huge width that
// then fails to allocate; here it is refused.
inline uint32_t need_count(const json &config, const std::string &key) {
    const int64_t v = need(config, key).template get<int64_t>();
    if (v < 0 || v > (int64_t)std::numeric_limits<uint32_t>::max())
        throw std::invalid_argument("n_frequencies and n_dims_to_encode must be non-negative 32-bit numbers");
    return (uint32_t)v;
}

template <typename T> Built<T> identity(const json &config, std::optional<uint32_t> padded, tnn::queue &q) {
    const float offset = need(config, EncodingParams::OFFSET);
    const float scale = need(config, EncodingParams::SCALE);
    const uint32_t dims = need(config, EncodingParams::N_DIMS_TO_ENCODE);
    return std::make_shared<IdentityEncoding<T>>(dims, padded.value_or(dims), scale, offset, q);
}

template <typename T> Built<T> spherical_harmonics(const json &config, std::optional<uint32_t> padded, tnn::queue &q) {
    const uint32_t degree = need(config, EncodingParams::DEGREE);
    const uint32_t dims = need(config, EncodingParams::N_DIMS_TO_ENCODE);
    return std::make_shared<SphericalHarmonicsEncoding<T>>(degree, dims, padded.value_or(degree * degree), q);
}

template <typename T> Built<T> frequency(const json &config, std::optional<uint32_t> padded, tnn::queue &q) {
    const uint32_t n_freq = need_count(config, EncodingParams::N_FREQUENCIES);
    const uint32_t dims = need_count(config, EncodingParams::N_DIMS_TO_ENCODE);
    if (n_freq == 0) throw std::invalid_argument("Output width cannot be zero");
    if (std::numeric_limits<uint32_t>::max() / n_freq < 2 * dims)
        throw std::invalid_argument("n_frequencies * 2 * n_dims_to_encode exceeds uint32_t max");
    return std::make_shared<FrequencyEncoding<T>>(n_freq, dims, padded.value_or(2 * n_freq * dims), q);
}

template <typename T> Built<T> grid(const json &config, std::optional<uint32_t> padded, tnn::queue &q) {
    static_assert(std::is_same<T, float>::value, "the grid encoding stores float parameters");
    return tinydpcppnn::encodings::grid::create_grid_encoding<T>(config, padded, q);
}

// Every key some encoding reads; anything else in a configuration earns a warning, not an error.
inline const std::array<const std::string *, 16> &known_keys() {
    static const std::array<const std::string *, 16> keys = {
        &EncodingParams::ENCODING,        &EncodingParams::N_DIMS_TO_ENCODE,     &EncodingParams::GRID_TYPE,
        &EncodingParams::N_LEVELS,        &EncodingParams::N_FEATURES,           &EncodingParams::N_FEATURES_PER_LEVEL,
        &EncodingParams::LOG2_HASHMAP_SIZE, &EncodingParams::BASE_RESOLUTION,    &EncodingParams::PER_LEVEL_SCALE,
        &EncodingParams::DEGREE,          &EncodingParams::SCALE,                &EncodingParams::OFFSET,
        &EncodingParams::HASH,            &EncodingParams::INTERPOLATION_METHOD, &EncodingParams::USE_STOCHASTIC_INTERPOLATION,
        &EncodingParams::N_FREQUENCIES};
    return keys;
}

inline void warn_about_unknown_keys(const json &config) {
    for (const auto &kv : config.items()) {
        bool known = false;
        for (const std::string *k : known_keys()) known = known || (*k == kv.first);
        if (known) continue;
        std::cout << "WARNING: found unknown option in encoding config. Please ensure that your options are one of the following:\n.";
        for (const std::string *k : known_keys()) std::cout << "\t" << *k << std::endl;
        return;
    }
}

} // namespace encoding_builders
} // namespace tnn

template <typename T>
std::shared_ptr<Encoding<T>> create_encoding(const json &config, tnn::queue &Q, std::optional<uint32_t> padded_output_width = std::nullopt) {
    namespace eb = tnn::encoding_builders;
    if (!config.contains(EncodingParams::ENCODING))
        throw std::invalid_argument("Config needs to contain encoding, key " + EncodingParams::ENCODING);
    const std::string name = config[EncodingParams::ENCODING];
    const std::pair<const std::string *, eb::Builder<T>> table[] = {{&EncodingNames::IDENTITY, &eb::identity<T>},
                                                                    {&EncodingNames::SPHERICALHARMONICS, &eb::spherical_harmonics<T>},
                                                                    {&EncodingNames::GRID, &eb::grid<T>},
                                                                    {&EncodingNames::FREQUENCY, &eb::frequency<T>}};
    for (const auto &entry : table) {
        if (*entry.first != name) continue;
        eb::warn_about_unknown_keys(config);
        return entry.second(config, padded_output_width, Q);
    }
    throw std::invalid_argument("Unknown encoding type: " + name);
}
