// create_encoding: configuration -> encoding object. Mirrors include/encodings/encoding_factory.h of the
// reference (factories :25-110, create_encoding with its key check :112-180).
#pragma once

#include <algorithm>
#include <iostream>
#include <limits>
#include <unordered_set>

#include "encoding.h"
#include "frequency.h"
#include "grid.h"
#include "identity.h"
#include "spherical_harmonics.h"

template <typename T> class EncodingFactory {
  public:
    virtual ~EncodingFactory() {}
    virtual std::shared_ptr<Encoding<T>> create(const json &config, std::optional<uint32_t> padded_output_width, tnn::queue &Q) const = 0;
};

template <typename T> class IdentityEncodingFactory : public EncodingFactory<T> {
  public:
    std::shared_ptr<Encoding<T>> create(const json &config, std::optional<uint32_t> padded_output_width, tnn::queue &Q) const override {
        if (!config.contains(EncodingParams::OFFSET)) throw std::invalid_argument("Config misses " + EncodingParams::OFFSET);
        if (!config.contains(EncodingParams::SCALE)) throw std::invalid_argument("Config misses " + EncodingParams::SCALE);
        if (!config.contains(EncodingParams::N_DIMS_TO_ENCODE)) throw std::invalid_argument("Config misses " + EncodingParams::N_DIMS_TO_ENCODE);
        const uint32_t n_dims_to_encode = config[EncodingParams::N_DIMS_TO_ENCODE];
        const float scale = config[EncodingParams::SCALE];
        const float offset = config[EncodingParams::OFFSET];
        return std::make_shared<IdentityEncoding<T>>(n_dims_to_encode, padded_output_width.has_value() ? padded_output_width.value() : n_dims_to_encode,
                                                     scale, offset, Q);
    }
};

template <typename T> class SphericalHarmonicsEncodingFactory : public EncodingFactory<T> {
  public:
    std::shared_ptr<Encoding<T>> create(const json &config, std::optional<uint32_t> padded_output_width, tnn::queue &Q) const override {
        if (!config.contains(EncodingParams::DEGREE)) throw std::invalid_argument("Config misses " + EncodingParams::DEGREE);
        if (!config.contains(EncodingParams::N_DIMS_TO_ENCODE)) throw std::invalid_argument("Config misses " + EncodingParams::N_DIMS_TO_ENCODE);
        const uint32_t degree = config[EncodingParams::DEGREE];
        const uint32_t n_dims_to_encode = config[EncodingParams::N_DIMS_TO_ENCODE];
        return std::make_shared<SphericalHarmonicsEncoding<T>>(
            degree, n_dims_to_encode, padded_output_width.has_value() ? padded_output_width.value() : (degree * degree), Q);
    }
};

template <typename T> class FrequencyEncodingFactory : public EncodingFactory<T> {
  public:
    std::shared_ptr<Encoding<T>> create(const json &config, std::optional<uint32_t> padded_output_width, tnn::queue &Q) const override {
        if (!config.contains(EncodingParams::N_FREQUENCIES)) throw std::invalid_argument("Config misses " + EncodingParams::N_FREQUENCIES);
        if (!config.contains(EncodingParams::N_DIMS_TO_ENCODE)) throw std::invalid_argument("Config misses " + EncodingParams::N_DIMS_TO_ENCODE);
        // negative values are rejected here; the reference lets them wrap to huge unsigned widths, which then fail to allocate
        const int64_t n_freq = config[EncodingParams::N_FREQUENCIES].template get<int64_t>();
        const int64_t n_dims = config[EncodingParams::N_DIMS_TO_ENCODE].template get<int64_t>();
        if (n_freq < 0 || n_dims < 0 || n_freq > 0xffffffffll || n_dims > 0xffffffffll)
            throw std::invalid_argument("n_frequencies and n_dims_to_encode must be non-negative 32-bit numbers");
        const uint32_t n_frequencies = (uint32_t)n_freq, n_dims_to_encode = (uint32_t)n_dims;
        if (n_frequencies == 0) throw std::invalid_argument("Output width cannot be zero");
        if (std::numeric_limits<uint32_t>::max() / n_frequencies < 2 * n_dims_to_encode)
            throw std::invalid_argument("n_frequencies * 2 * n_dims_to_encode exceeds uint32_t max");
        return std::make_shared<FrequencyEncoding<T>>(
            n_frequencies, n_dims_to_encode,
            padded_output_width.has_value() ? padded_output_width.value() : 2 * n_frequencies * n_dims_to_encode, Q);
    }
};

template <typename T> class GridEncodingFactory : public EncodingFactory<T> {
  public:
    std::shared_ptr<Encoding<T>> create(const json &config, std::optional<uint32_t> padded_output_width, tnn::queue &Q) const override {
        static_assert(std::is_same<T, float>::value, "GridEncodingFactory only supports float");
        return tinydpcppnn::encodings::grid::create_grid_encoding<T>(config, padded_output_width, Q);
    }
};

template <typename T>
std::shared_ptr<Encoding<T>> create_encoding(const json &config, tnn::queue &Q, std::optional<uint32_t> padded_output_width = std::nullopt) {
    if (!config.contains(EncodingParams::ENCODING))
        throw std::invalid_argument("Config needs to contain encoding, key " + EncodingParams::ENCODING);
    const std::string name = config[EncodingParams::ENCODING];
    if (name != EncodingNames::IDENTITY && name != EncodingNames::SPHERICALHARMONICS && name != EncodingNames::GRID &&
        name != EncodingNames::FREQUENCY)
        throw std::invalid_argument("Unknown encoding type: " + name);

    const std::unordered_set<std::string> valid_keys(
        {EncodingParams::ENCODING, EncodingParams::N_DIMS_TO_ENCODE, EncodingParams::GRID_TYPE, EncodingParams::N_LEVELS,
         EncodingParams::N_FEATURES, EncodingParams::N_FEATURES_PER_LEVEL, EncodingParams::LOG2_HASHMAP_SIZE, EncodingParams::BASE_RESOLUTION,
         EncodingParams::PER_LEVEL_SCALE, EncodingParams::DEGREE, EncodingParams::SCALE, EncodingParams::OFFSET, EncodingParams::HASH,
         EncodingParams::INTERPOLATION_METHOD, EncodingParams::USE_STOCHASTIC_INTERPOLATION, EncodingParams::N_FREQUENCIES});
    const bool valid = std::all_of(config.items().begin(), config.items().end(),
                                   [&valid_keys](const auto &kv) { return valid_keys.count(kv.first) != 0; });
    if (!valid) {
        std::cout << "WARNING: found unknown option in encoding config. Please ensure that your options are one of the following:\n.";
        for (const auto &k : valid_keys) std::cout << "\t" << k << std::endl;
    }

    std::unique_ptr<EncodingFactory<T>> factory;
    if (name == EncodingNames::IDENTITY)
        factory = std::make_unique<IdentityEncodingFactory<T>>();
    else if (name == EncodingNames::SPHERICALHARMONICS)
        factory = std::make_unique<SphericalHarmonicsEncodingFactory<T>>();
    else if (name == EncodingNames::GRID)
        factory = std::make_unique<GridEncodingFactory<T>>();
    else
        factory = std::make_unique<FrequencyEncodingFactory<T>>();
    return factory->create(config, padded_output_width, Q);
}
