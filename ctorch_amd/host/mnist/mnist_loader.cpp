// IDX files as the reference reads them (mnist/mnist_loader.cpp:7-73): big-endian header words,
// magic 2051 (images: count, rows, cols) or 2049 (labels: count), then one unsigned byte per
// pixel / label.  A short file is an error here (the reference reads garbage past the end).
#include "mnist_loader.h"

#include <cstdint>
#include <cstdio>
#include <stdexcept>

#include "kernels.h"

namespace {

struct File {
    FILE* f;
    explicit File(const std::string& path) : f(std::fopen(path.c_str(), "rb")) {
        if (!f) throw std::runtime_error("cannot open file: " + path);
    }
    ~File() { std::fclose(f); }
    int32_t be32() {
        unsigned char b[4];
        if (std::fread(b, 1, 4, f) != 4) throw std::runtime_error("IDX header is truncated");
        return int32_t((uint32_t(b[0]) << 24) | (uint32_t(b[1]) << 16) | (uint32_t(b[2]) << 8) | uint32_t(b[3]));
    }
    std::vector<unsigned char> bytes(size_t n) {
        std::vector<unsigned char> v(n);
        if (n && std::fread(v.data(), 1, n, f) != n) throw std::runtime_error("IDX payload is truncated");
        return v;
    }
};

}  // namespace

MNISTLoader::MNISTLoader(const std::string& dir) : data_dir(dir) {}

std::vector<unsigned char> MNISTLoader::read_images(const std::string& filename, int& num_images, int& rows, int& cols) {
    File file(data_dir + "/" + filename);
    if (file.be32() != 2051) throw std::runtime_error("not an IDX image file: " + filename);
    num_images = file.be32();
    rows = file.be32();
    cols = file.be32();
    if (num_images < 0 || rows < 0 || cols < 0) throw std::runtime_error("negative IDX dimension: " + filename);
    return file.bytes(size_t(num_images) * size_t(rows) * size_t(cols));
}

std::vector<unsigned char> MNISTLoader::read_labels(const std::string& filename, int& num_labels) {
    File file(data_dir + "/" + filename);
    if (file.be32() != 2049) throw std::runtime_error("not an IDX label file: " + filename);
    num_labels = file.be32();
    if (num_labels < 0) throw std::runtime_error("negative IDX dimension: " + filename);
    return file.bytes(size_t(num_labels));
}

void MNISTLoader::load(const std::string& image_file, const std::string& label_file, Tensor& images, Tensor& labels) {
    int n = 0, rows = 0, cols = 0, nl = 0;
    std::vector<unsigned char> px = read_images(image_file, n, rows, cols);
    std::vector<unsigned char> lb = read_labels(label_file, nl);
    images = ctorch_amd_host::unit_from_bytes(px.data(), size_t(n), size_t(rows) * size_t(cols));   // pixel / 255.0f
    std::vector<float> lf(lb.begin(), lb.end());
    labels = Tensor::from_host(lf.data(), {size_t(nl)}, DeviceType::kAMD);
}

void MNISTLoader::load_training_data(Tensor& images, Tensor& labels) {
    load("train-images-idx3-ubyte", "train-labels-idx1-ubyte", images, labels);
}

void MNISTLoader::load_test_data(Tensor& images, Tensor& labels) {
    load("t10k-images-idx3-ubyte", "t10k-labels-idx1-ubyte", images, labels);
}
