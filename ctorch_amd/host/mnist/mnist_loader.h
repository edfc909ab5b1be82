// MNIST IDX loader with the reference's interface (mnist/mnist_loader.h:9-26): same class, same
// two load calls, same tensor shapes ([images, rows*cols] fp32 pixels in [0, 1], [images] fp32
// labels).  The tensors come back resident on the MI355X: the files are read in bulk, the pixel
// bytes are uploaded as bytes (a quarter of the fp32 size) and converted by a device kernel.
#ifndef CTORCH_AMD_HOST_MNIST_LOADER_H
#define CTORCH_AMD_HOST_MNIST_LOADER_H

#include <string>
#include <vector>

#include "Tensor.h"

class MNISTLoader {
   public:
    explicit MNISTLoader(const std::string& dir);
    void load_training_data(Tensor& images, Tensor& labels);
    void load_test_data(Tensor& images, Tensor& labels);

   private:
    std::string data_dir;
    std::vector<unsigned char> read_images(const std::string& filename, int& num_images, int& rows, int& cols);
    std::vector<unsigned char> read_labels(const std::string& filename, int& num_labels);
    void load(const std::string& image_file, const std::string& label_file, Tensor& images, Tensor& labels);
};

#endif
