// Files the host classes read and write: encoding configurations (json) and flat lists of numbers (network weights).
//
// Takes the place of the part of the reference's include/common/io.h that lies on the path: loadJsonConfig (:43-60),
// validateAndCopyEncodingConfig (:62-79), load_weights_as_packed_from_file (:81-107), loadVectorFromCSV / saveCSV
// (:109-138). Its image, target-vector and matrix-printing helpers serve the reference's samples and are not provided.
//
// Number files: text, one number after another, separated by any mix of newlines, commas, semicolons and blanks
// (the reference writes one per line and reads either one per line or comma-separated). Anything else in the file is an
// error that names the file and the place; a file that cannot be opened is an error too.
#pragma once

#include <cstdlib>
#include <fstream>
#include <iterator>
#include <limits>
#include <stdexcept>
#include <string>
#include <vector>

#include "encoding.h"

namespace io {

namespace detail {

inline std::string file_contents(const std::string &path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::invalid_argument("cannot open '" + path + "' for reading");
    return std::string(std::istreambuf_iterator<char>(in), std::istreambuf_iterator<char>());
}

inline bool separates_numbers(char c) { return c == '\n' || c == '\r' || c == ',' || c == ';' || c == ' ' || c == '\t'; }

/// Every number of `text` in order. `origin` only appears in error messages.
inline std::vector<float> numbers_of(const std::string &text, const std::string &origin) {
    std::vector<float> out;
    const char *const begin = text.c_str(), *const end = begin + text.size();
    for (const char *p = begin; p < end;) {
        if (separates_numbers(*p)) {
            ++p;
            continue;
        }
        char *after = nullptr;
        const double v = std::strtod(p, &after);
        if (after == p || (after < end && !separates_numbers(*after)))
            throw std::invalid_argument(origin + ": not a number at byte " + std::to_string(p - begin));
        // too large for a float, whether or not it fits a double (a text "inf" passes: it says what it means)
        const bool spelled_inf = std::string(p, static_cast<size_t>(after - p)).find_first_of("nN") != std::string::npos;
        if (!spelled_inf && (v > std::numeric_limits<float>::max() || v < -std::numeric_limits<float>::max()))
            throw std::out_of_range(origin + ": number out of range at byte " + std::to_string(p - begin));
        out.push_back(static_cast<float>(v));
        p = after;
    }
    return out;
}

struct EnumName {
    const char *name;
    int ordinal;
};

// The spellings a configuration may use for the enum-valued keys of a grid encoding (include/encodings/encoding.h of
// the reference, :28-90), with the ordinal the encoding factory reads.
inline constexpr EnumName kGridTypeNames[] = {{"Hash", (int)GridType::Hash}, {"Dense", (int)GridType::Dense}, {"Tiled", (int)GridType::Tiled}};
inline constexpr EnumName kHashNames[] = {{"Prime", (int)HashType::Prime},
                                          {"CoherentPrime", (int)HashType::CoherentPrime},
                                          {"ReversedPrime", (int)HashType::ReversedPrime},
                                          {"Rng", (int)HashType::Rng}};
inline constexpr EnumName kInterpolationNames[] = {{"Nearest", (int)InterpolationType::Nearest},
                                                   {"Linear", (int)InterpolationType::Linear},
                                                   {"Smoothstep", (int)InterpolationType::Smoothstep}};

template <size_t N> int ordinal_of(const EnumName (&names)[N], const std::string &spelled, const std::string &key) {
    for (const EnumName &e : names)
        if (spelled == e.name) return e.ordinal;
    throw std::runtime_error("Invalid enum value '" + spelled + "' for '" + key + "'");
}

} // namespace detail

/// A copy of `config` in which the enum-valued keys that are spelled out as strings hold the enum's ordinal, which is
/// what create_encoding reads. Keys that are absent or already numeric stay as they are.
inline json validateAndCopyEncodingConfig(const json &config) {
    json out = config;
    auto settle = [&out](const std::string &key, const auto &names) {
        if (out.contains(key) && out[key].is_string()) out[key] = json(detail::ordinal_of(names, out[key].template get<std::string>(), key));
    };
    settle(EncodingParams::GRID_TYPE, detail::kGridTypeNames);
    settle(EncodingParams::HASH, detail::kHashNames);
    settle(EncodingParams::INTERPOLATION_METHOD, detail::kInterpolationNames);
    return out;
}

inline json loadJsonConfig(const std::string &filename) {
    std::string text;
    try {
        text = detail::file_contents(filename);
    } catch (const std::invalid_argument &) {
        throw std::runtime_error("Error: Unable to open file '" + filename + "'");
    }
    return validateAndCopyEncodingConfig(json::parse(text));
}

/// The numbers of a file as T, in file order.
template <typename T> std::vector<T> loadVectorFromCSV(const std::string &filename) {
    const std::vector<float> values = detail::numbers_of(detail::file_contents(filename), filename);
    std::vector<T> out(values.size());
    for (size_t i = 0; i < values.size(); ++i) out[i] = static_cast<T>(values[i]);
    return out;
}

/// One number per line, with the digits a float needs to survive the round trip.
template <typename T> void saveCSV(const std::string &filename, const std::vector<T> &data) {
    std::ofstream out(filename);
    if (!out) throw std::invalid_argument("cannot open '" + filename + "' for writing");
    out.precision(std::numeric_limits<float>::max_digits10);
    for (const T &v : data) out << static_cast<float>(v) << '\n';
    if (!out.flush()) throw std::runtime_error("writing '" + filename + "' failed");
}

/// A weight file holds the network's matrices unpacked, [in][out] row-major, first matrix first: input_width x WIDTH, then
/// n_hidden_layers - 1 of WIDTH x WIDTH, then WIDTH x output_width (what Network::get_weights_matrices, unpacked, would
/// list). Returns them in the packed parameter layout that set_weights_matrices(v, /*packed=*/true) takes.
template <typename T, int WIDTH>
std::vector<T> load_weights_as_packed_from_file(const std::string &filename, int n_hidden_layers, int input_width, int output_width) {
    std::vector<T> unpacked = loadVectorFromCSV<T>(filename);
    const size_t expected = (size_t)WIDTH * ((size_t)input_width + (size_t)output_width) +
                            (size_t)(n_hidden_layers > 0 ? n_hidden_layers - 1 : 0) * WIDTH * WIDTH;
    if (unpacked.size() != expected)
        throw std::invalid_argument(filename + ": " + std::to_string(unpacked.size()) + " values, the network has " + std::to_string(expected));
    return get_packed_weights<T>(unpacked, n_hidden_layers, input_width, WIDTH, output_width);
}

} // namespace io
