// create_encoding: configuration -> encoding object. Mirrors include/encodings/encoding_factory.h of the
// reference (factories :25-110, create_encoding with its key check :112-180).
#pragma once

#include <algorithm>
#include <iostream>
#include <unordered_set>

#include "encoding.h"
#include "grid.h"

template <typename T> class EncodingFactory {
  public:
    virtual ~EncodingFactory() {}
    virtual std::shared_ptr<Encoding<T>> create(const json &config, std::optional<uint32_t> padded_output_width, tnn::queue &Q) const = 0;
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
    if (name == EncodingNames::GRID)
        factory = std::make_unique<GridEncodingFactory<T>>();
    else
        throw std::invalid_argument("Encoding type " + name + " is not part of this build; only " + EncodingNames::GRID + " is.");
    return factory->create(config, padded_output_width, Q);
}
