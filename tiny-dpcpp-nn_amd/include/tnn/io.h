// Configuration and weight file helpers. Mirrors include/common/io.h of the reference: the string -> enum
// maps (:14-31), stringToEnum (:33-41), loadJsonConfig (:43-60), validateAndCopyEncodingConfig (:62-79),
// load_weights_as_packed_from_file (:81-107), loadVectorFromCSV / saveCSV (:109-138), loadCSV (:140-156),
// readTargetVectorsFromFile (:158-185), saveImageToPGM (:187-200), printDeviceMatrix (:202-221).
#pragma once

#include <fstream>
#include <iostream>
#include <sstream>
#include <unordered_map>

#include "encoding.h"

namespace io {

inline const std::unordered_map<std::string, GridType> gridTypeMap{{"Hash", GridType::Hash}, {"Dense", GridType::Dense}, {"Tiled", GridType::Tiled}};
inline const std::unordered_map<std::string, HashType> hashTypeMap{
    {"Prime", HashType::Prime}, {"CoherentPrime", HashType::CoherentPrime}, {"ReversedPrime", HashType::ReversedPrime}, {"Rng", HashType::Rng}};
inline const std::unordered_map<std::string, InterpolationType> interpolationTypeMap{
    {"Nearest", InterpolationType::Nearest}, {"Linear", InterpolationType::Linear}, {"Smoothstep", InterpolationType::Smoothstep}};
inline const std::unordered_map<std::string, GradientMode> gradientModeMap{
    {"Ignore", GradientMode::Ignore}, {"Overwrite", GradientMode::Overwrite}, {"Accumulate", GradientMode::Accumulate}};
inline const std::unordered_map<std::string, ReductionType> reductionTypeMap{
    {"Concatenation", ReductionType::Concatenation}, {"Sum", ReductionType::Sum}, {"Product", ReductionType::Product}};

template <typename T> T stringToEnum(const std::string &value, const std::unordered_map<std::string, T> &enumMap) {
    const auto it = enumMap.find(value);
    if (it != enumMap.end()) return it->second;
    throw std::runtime_error("Invalid enum value");
}

/// Returns a copy of the configuration in which the enum-valued keys given as strings hold the enum ordinals.
inline json validateAndCopyEncodingConfig(const json &encodingConfig) {
    json copy = encodingConfig;
    auto convertIfString = [&copy](const auto &enumMap, const std::string &key) {
        if (copy.contains(key) && copy[key].is_string()) copy[key] = json(stringToEnum(copy[key].template get<std::string>(), enumMap));
    };
    convertIfString(gridTypeMap, EncodingParams::GRID_TYPE);
    convertIfString(hashTypeMap, EncodingParams::HASH);
    convertIfString(interpolationTypeMap, EncodingParams::INTERPOLATION_METHOD);
    return copy;
}

inline json loadJsonConfig(const std::string &filename) {
    std::ifstream file{filename};
    if (!file) throw std::runtime_error("Error: Unable to open file '" + filename + "'");
    std::stringstream buffer;
    buffer << file.rdbuf();
    return validateAndCopyEncodingConfig(json::parse(buffer.str()));
}

/// One value per line, the flat list of unpacked [in][out] matrices -> packed parameters.
template <typename T, int WIDTH>
std::vector<T> load_weights_as_packed_from_file(std::string filename, int m_n_hidden_layers, int input_width, int output_width) {
    std::vector<T> data_vec;
    std::ifstream file(filename);
    if (!file.is_open()) std::cerr << "Error opening file: " << filename << std::endl;
    std::string line;
    while (std::getline(file, line)) {
        try {
            data_vec.push_back((T)(float)std::stod(line));
        } catch (const std::invalid_argument &e) {
            std::cerr << "Invalid argument: " << e.what() << std::endl;
        } catch (const std::out_of_range &e) {
            std::cerr << "Out of range: " << e.what() << std::endl;
        }
    }
    return get_packed_weights<T>(data_vec, m_n_hidden_layers, input_width, WIDTH, output_width);
}

template <typename T> std::vector<T> loadVectorFromCSV(const std::string &filename) {
    std::vector<T> data;
    std::ifstream file(filename);
    if (!file.is_open()) throw std::invalid_argument("Failed to open the file for reading: " + filename);
    std::string line;
    while (std::getline(file, line)) {
        std::istringstream ss(line);
        std::string token;
        while (std::getline(ss, token, ',')) data.push_back(static_cast<T>(std::stof(token)));
    }
    return data;
}

template <typename T> void saveCSV(const std::string &filename, const std::vector<T> &data) {
    std::ofstream file(filename);
    if (!file.is_open()) throw std::invalid_argument("Failed to open the file for writing: " + filename);
    for (const auto &value : data) file << (float)value << std::endl;
}

/// One float per line (what saveCSV writes); a file that cannot be opened gives an empty vector, as in the reference
/// (include/common/io.h:140-156).
inline std::vector<float> loadCSV(const std::string &filename) {
    std::vector<float> data;
    std::ifstream file(filename);
    std::string line;
    while (file.is_open() && std::getline(file, line)) {
        float value = 0.0f;
        std::istringstream(line) >> value;
        data.push_back(value);
    }
    return data;
}

/// One vector per line, values separated by `delimiter` (include/common/io.h:158-185). A file that cannot be opened is
/// reported on stderr and gives no vectors.
inline std::vector<std::vector<float>> readTargetVectorsFromFile(const std::string &filename, char delimiter) {
    std::vector<std::vector<float>> vectors;
    std::ifstream file(filename);
    if (!file.is_open()) {
        std::cerr << "Error opening " << filename << std::endl;
        return vectors;
    }
    std::string line, token;
    while (std::getline(file, line)) {
        std::vector<float> row;
        std::istringstream ss(line);
        while (std::getline(ss, token, delimiter)) row.push_back((float)std::stod(token));
        vectors.push_back(std::move(row));
    }
    return vectors;
}

/// Binary greyscale image ("P5", 8 bits per pixel), include/common/io.h:187-200.
inline void saveImageToPGM(const std::string &filename, const int width, const int height, const std::vector<unsigned char> &image) {
    std::ofstream file(filename, std::ios::out | std::ios::binary);
    file << "P5\n" << width << " " << height << "\n255\n";
    file.write(reinterpret_cast<const char *>(image.data()), (std::streamsize)image.size());
}

/// Copies every matrix behind the view to the host and prints the values, with a separator line after every
/// `line_break_every` of them (include/common/io.h:202-221; the queue is the HIP stream wrapper here).
template <typename T> void printDeviceMatrix(const DeviceMatricesView<T> &view, tnn::queue &q, int line_break_every) {
    const size_t n = view.nelements();
    std::vector<T> host(n);
    q.wait();
    tnn::hip_check(hipMemcpy(host.data(), view.GetMatrixPointer(0), n * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy");
    for (size_t i = 0; i < n; ++i) {
        std::cout << (float)host[i] << ", ";
        if (line_break_every > 0 && (i + 1) % (size_t)line_break_every == 0) std::cout << "========================" << std::endl;
    }
}

} // namespace io
