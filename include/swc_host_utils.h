/*
 * swc_host_utils.h — host-side helpers of programs generated for the HIP
 * target: tensor file IO, host initialisers, printing and the accuracy counter.
 * They play the part of the reference's src/codegen/utils/image.h (load/store,
 * :13-51) and of the initialiser / print / accuracy helpers at the edges of
 * src/codegen/utils/kernels.h (:11-29, :615-639), with the same names and
 * argument order, so that generated call sites read the same on both targets.
 * File format: raw little-endian elements, `offset` counted in elements.
 */
#ifndef SWC_HOST_UTILS_H_
#define SWC_HOST_UTILS_H_

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <random>
#include <string>

template <typename T> inline unsigned load(T *data, size_t size, size_t offset, const std::string &path) {
    std::FILE *f = std::fopen(path.c_str(), "rb");
    if (!f || std::fseek(f, (long)(offset * sizeof(T)), SEEK_SET) != 0 || std::fread(data, sizeof(T), size, f) != size) {
        std::cout << "Error loading " << path << "\n";
        std::exit(EXIT_FAILURE);
    }
    std::fclose(f);
    return (unsigned)size;
}

template <typename T> inline void store(const T *data, size_t size, const std::string &path) {
    std::FILE *f = std::fopen(path.c_str(), "wb");
    if (!f || std::fwrite(data, sizeof(T), size, f) != size) {
        std::cout << "Error opening " << path << "\n";
        std::exit(EXIT_FAILURE);
    }
    std::fclose(f);
}

template <typename T> inline void initTensorConstant(T *data, size_t size, float value) {
    for (size_t i = 0; i < size; ++i) data[i] = (T)value;
}
template <typename T> inline void initTensorZero(T *data, size_t size) { initTensorConstant(data, size, 0.f); }

// uniform in +-sqrt(3/filterSize), seeded from the system entropy source
template <typename T> inline void initTensorXavier(T *data, size_t size, float filterSize) {
    std::random_device entropy;
    std::mt19937 gen(entropy());
    const double bound = std::sqrt(3.0 / (double)filterSize);
    std::uniform_real_distribution<double> dist(-bound, bound);
    for (size_t i = 0; i < size; ++i) data[i] = (T)dist(gen);
}

// fixed notation, three decimals, one row per line
template <typename T> inline void printMatrix(const T *a, int m, int n) {
    std::cout.setf(std::ios::fixed);
    std::cout.precision(3);
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) std::cout << a[(size_t)i * n + j] << " ";
        std::cout << std::endl;
    }
}

// accum[0] += rows whose label appears among their n predictions; accum[1] += rows
inline void accuracy_i(const int *pred, const int *label, int *accum, int m, int n) {
    for (int i = 0; i < m; ++i) {
        ++accum[1];
        for (int j = 0; j < n; ++j)
            if (pred[(size_t)i * n + j] == label[i]) {
                ++accum[0];
                break;
            }
    }
}

#endif /* SWC_HOST_UTILS_H_ */
