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
#include <cstring>
#include <iostream>
#include <initializer_list>
#include <random>
#include <string>
#include <vector>

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

// Record reader of the generated batch loop: a file of `sample_num` records
// <label><data>, where a label is one byte (ONE_BYTE_AS_INT) or a 4-byte float
// read as an integer class (FOUR_BYTES_AS_FLOAT), and data elements are bytes or
// 4-byte floats likewise.  next() fills one mini-batch (label_shape[0] records)
// and returns false once `epochs` passes over the file are done; a mini-batch
// that reaches the end of the file goes on with the first records of the next
// pass, and what is left of the last pass is dropped.  A byte is read as the
// reference reads it, through `char` (values above 127 come out negative).
// Same constructor and next()/shift() as the reference's
// src/codegen/utils/DataLoader.h:56-63 (DataLoader.cpp:98-168).
#ifndef SWC_BYTES_PROTO_DEFINED
#define SWC_BYTES_PROTO_DEFINED
enum BytesProto { ONE_BYTE_AS_INT, FOUR_BYTES_AS_FLOAT };
#endif

class DataLoader {
    std::FILE *file_{nullptr};
    std::string path_;
    BytesProto labelProto_, dataProto_;
    size_t epochs_, samples_, batch_, dataPerSample_{1};
    size_t cursor_{0}, epoch_{0};
    std::vector<unsigned char> raw_;

    static size_t width(BytesProto p) { return p == ONE_BYTE_AS_INT ? 1 : 4; }
    void rewindFile() {
        std::rewind(file_);
        cursor_ = 0;
    }
    template <typename T> static void decode(const unsigned char *src, BytesProto p, size_t n, T *dst) {
        for (size_t i = 0; i < n; ++i) {
            if (p == ONE_BYTE_AS_INT) {
                dst[i] = (T)(signed char)src[i];
            } else {
                float f;
                std::memcpy(&f, src + 4 * i, 4);
                dst[i] = (T)f;
            }
        }
    }

  public:
    DataLoader(const std::string &filename, BytesProto label_proto, BytesProto data_proto, size_t epochs,
               size_t sample_num, const std::initializer_list<size_t> &label_shape,
               const std::initializer_list<size_t> &data_shape)
        : path_(filename), labelProto_(label_proto), dataProto_(data_proto), epochs_(epochs), samples_(sample_num),
          batch_(*label_shape.begin()) {
        size_t i = 0;
        for (size_t d : data_shape)
            if (i++ > 0) dataPerSample_ *= d;
        file_ = std::fopen(path_.c_str(), "rb");
        if (!file_) {
            std::cout << "Error loading " << path_ << "\n";
            std::exit(EXIT_FAILURE);
        }
        raw_.resize(width(labelProto_) + width(dataProto_) * dataPerSample_);
    }
    ~DataLoader() {
        if (file_) std::fclose(file_);
    }
    DataLoader(const DataLoader &) = delete;
    DataLoader &operator=(const DataLoader &) = delete;

    bool next(int *label_batch, float *data_batch) {
        if (epoch_ >= epochs_) return false;
        for (size_t s = 0; s < batch_; ++s) {
            if (cursor_ == samples_) {   // the mini-batch goes on with the first records of the next epoch
                ++epoch_;
                rewindFile();
                if (epoch_ >= epochs_ || samples_ == 0) return false;
            }
            if (std::fread(raw_.data(), 1, raw_.size(), file_) != raw_.size()) return false;
            decode(raw_.data(), labelProto_, 1, label_batch + s);
            decode(raw_.data() + width(labelProto_), dataProto_, dataPerSample_, data_batch + s * dataPerSample_);
            ++cursor_;
        }
        return true;
    }
    // continue as if n mini-batches had been read since the start (a run restored from a snapshot): epoch and
    // position follow from n, as in the reference's DataLoader.cpp:161-168.  (There the file is opened by the
    // first next(), so a shift before it — where the generated program has it — leaves the file position at the
    // start while the counters move; here both move.)
    void shift(size_t n) {
        const size_t seen = n * batch_;
        epoch_ = samples_ ? seen / samples_ : 0;
        cursor_ = samples_ ? seen % samples_ : 0;
        std::fseek(file_, (long)(cursor_ * raw_.size()), SEEK_SET);
    }
};

#endif /* SWC_HOST_UTILS_H_ */
