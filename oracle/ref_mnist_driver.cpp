// TEST INFRASTRUCTURE ONLY.  A plain-C doorway into the reference's MNIST demo, next to
// ref_driver.cpp: the reference's own loader (mnist/mnist_loader.cpp) and the free functions of
// its demo program (mnist/mnist.cpp, compiled with its main() renamed) are linked into
// oracle/_ref/libctorch_ref.so from where they lie; nothing of them is copied here.
//
// This file and those two are compiled WITHOUT optimisation flags, as the reference's build does
// for its MnistTest target (CMakeLists.txt:56; -O3 -march=native are set on the library target
// only, :65-86): the optimiser update below is then a rounded product followed by a rounded
// difference, as in the reference's binary.
#include "mnist_loader.h"
#include "AutoDiff.h"
#include "Ctorch_Error.h"

#include <unistd.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

// free functions defined in the reference's mnist/mnist.cpp
float calculate_accuracy(const Tensor& y_pred, const Tensor& y_true);
void get_batch(const Tensor& images, const Tensor& labels, int batch_size, int batch_idx, Tensor& batch_images,
               Tensor& batch_labels);
int ctorch_reference_mnist_main();

namespace {

Tensor host_tensor(const float* src, std::vector<size_t> shape) {
    Tensor t(ShapeTag{}, shape, DType::kFloat, DeviceType::kCPU);
    if (src && t.numel()) std::memcpy(t.data<float>(), src, t.numel() * sizeof(float));
    return t;
}

}  // namespace

extern "C" {

// The reference's loader on the files in `dir`.  which: 1 = training files, 0 = test files.
// dims_out = {images, pixels per image}.  With null outputs only the dimensions are reported.
long ref_mnist_load(const char* dir, int which, float* images_out, float* labels_out, long* dims_out) {
    try {
        MNISTLoader loader(dir);
        Tensor images, labels;
        if (which) loader.load_training_data(images, labels);
        else loader.load_test_data(images, labels);
        dims_out[0] = static_cast<long>(images.shape()[0]);
        dims_out[1] = static_cast<long>(images.shape()[1]);
        if (images_out) std::memcpy(images_out, images.data<float>(), images.numel() * sizeof(float));
        if (labels_out) std::memcpy(labels_out, labels.data<float>(), labels.numel() * sizeof(float));
        return static_cast<long>(labels.numel());
    } catch (const std::exception&) {
        return -1;
    }
}

// mnist/mnist.cpp's calculate_accuracy on [rows, 10] predictions.
float ref_mnist_accuracy(const float* pred, const float* labels, long rows) {
    Tensor p = host_tensor(pred, {static_cast<size_t>(rows), 10});
    Tensor y = host_tensor(labels, {static_cast<size_t>(rows)});
    return calculate_accuracy(p, y);
}

// mnist/mnist.cpp's get_batch: rows [idx*batch, min((idx+1)*batch, n)) of images and labels.
long ref_mnist_get_batch(const float* images, const float* labels, long n, long pixels, long batch, long idx,
                         float* images_out, float* labels_out) {
    Tensor im = host_tensor(images, {static_cast<size_t>(n), static_cast<size_t>(pixels)});
    Tensor lb = host_tensor(labels, {static_cast<size_t>(n)});
    Tensor bi, bl;
    get_batch(im, lb, static_cast<int>(batch), static_cast<int>(idx), bi, bl);
    std::memcpy(images_out, bi.data<float>(), bi.numel() * sizeof(float));
    std::memcpy(labels_out, bl.data<float>(), bl.numel() * sizeof(float));
    return static_cast<long>(bl.numel());
}

// The demo's weight initialisation (mnist/mnist.cpp:21-27, :226 srand(42)) for one matrix:
// uniform in +-sqrt(1/fan_in) from the C library's rand().  `reseed` != 0 calls srand(seed) first.
void ref_mnist_xavier(float* w, long n, long fan_in, int reseed, unsigned seed) {
    if (reseed) srand(seed);
    float scale = std::sqrt(1.0f / fan_in);
    for (long i = 0; i < n; ++i) {
        float r = (2.0f * rand() / static_cast<float>(RAND_MAX)) - 1.0f;
        w[i] = r * scale;
    }
}

// The demo's training loop over the reference library, `steps` consecutive batches with batch
// index step % (n_images / batch), all inside one autograd context as the demo's main() has it:
// per step the calls of NeuralNetwork::train_step (mnist/mnist.cpp:44-84) and update_parameters
// (:86-93) in their order.  Parameters are updated in place; losses_out[s] is the loss of step s.
long ref_mnist_train(const float* images, const float* labels, long n_images, long I, long H1, long H2, long C,
                     float* W1p, float* b1p, float* W2p, float* b2p, float* W3p, float* b3p, long batch,
                     long steps, float lr, float* losses_out) {
    try {
        const size_t uI = I, uH1 = H1, uH2 = H2, uC = C;
        Tensor all_images = host_tensor(images, {static_cast<size_t>(n_images), uI});
        Tensor all_labels = host_tensor(labels, {static_cast<size_t>(n_images)});
        Tensor W1 = host_tensor(W1p, {uI, uH1}), b1 = host_tensor(b1p, {uH1});
        Tensor W2 = host_tensor(W2p, {uH1, uH2}), b2 = host_tensor(b2p, {uH2});
        Tensor W3 = host_tensor(W3p, {uH2, uC}), b3 = host_tensor(b3p, {uC});
        Tensor* params[6] = {&W1, &b1, &W2, &b2, &W3, &b3};
        const long num_batches = n_images / batch;
        AutoDiff autodiff;
        AutoDiffContext::Guard guard(&autodiff);
        for (long s = 0; s < steps; ++s) {
            Tensor x, y;
            get_batch(all_images, all_labels, static_cast<int>(batch), static_cast<int>(s % num_batches), x, y);
            x.requires_grad(false);
            y.requires_grad(false);
            for (Tensor* p : params) AutoDiffContext::current()->make_leaf(*p, true);
            for (Tensor* p : params) p->requires_grad(true);
            for (Tensor* p : params) AutoDiffContext::current()->zero_grad(*p);
            Tensor h1 = (x.matmul(W1) + b1).relu();
            Tensor h2 = (h1.matmul(W2) + b2).relu();
            Tensor logits = h2.matmul(W3) + b3;
            Tensor onehot(ShapeTag{}, {y.numel(), uC}, DType::kFloat, DeviceType::kCPU);
            for (size_t i = 0; i < y.numel(); ++i) {
                int lab = static_cast<int>(y.data<float>()[i]);
                for (size_t j = 0; j < uC; ++j) onehot.data<float>()[i * uC + j] = (static_cast<int>(j) == lab) ? 1.0f : 0.0f;
            }
            Tensor loss = logits.cross_entropy(onehot);
            losses_out[s] = loss.item<float>();
            backward(loss);
            for (Tensor* p : params) {
                Tensor g = grad(*p);
                float* w = p->data<float>();
                const float* gp = g.data<float>();
                for (size_t i = 0; i < p->numel(); ++i) w[i] -= gp[i] * lr;
            }
        }
        float* outs[6] = {W1p, b1p, W2p, b2p, W3p, b3p};
        for (int k = 0; k < 6; ++k) std::memcpy(outs[k], params[k]->data<float>(), params[k]->numel() * sizeof(float));
        return steps;
    } catch (const std::exception&) {
        return -1;
    }
}

// Runs the reference demo's own main() with `dir` as the working directory (it reads the four
// IDX files from "." and prints its epoch losses and accuracies to stdout).
int ref_mnist_main_in(const char* dir) {
    char old[4096];
    if (!getcwd(old, sizeof(old))) return -100;
    if (chdir(dir) != 0) return -101;
    int rc = ctorch_reference_mnist_main();
    if (chdir(old) != 0) return -102;
    return rc;
}

}  // extern "C"
