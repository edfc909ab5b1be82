// The model of the reference's MNIST demo (class NeuralNetwork, mnist/mnist.cpp:9-131) over device
// tensors: 784 -> hidden1 (ReLU) -> hidden2 (ReLU) -> 10, sum-reduced cross entropy on one-hot
// targets, plain SGD.  Same call order per step as the reference's train_step (:44-84); the host
// loops of the reference (one-hot targets, parameter update, prediction softmax, accuracy) are
// device launches, and a batch is a view of the resident data set instead of a copy.
#ifndef CTORCH_AMD_HOST_MNIST_MODEL_H
#define CTORCH_AMD_HOST_MNIST_MODEL_H

#include <cmath>
#include <cstdlib>
#include <vector>

#include "AutoDiff.h"
#include "Tensor.h"
#include "kernels.h"

class NeuralNetwork {
   public:
    Tensor W1, b1, W2, b2, W3, b3;
    float learning_rate;

    // Weights uniform in +-sqrt(1/fan_in) from the C library's rand() in the reference's order
    // (W1, W2, W3; mnist/mnist.cpp:21-27, :33-35), biases zero; generated on the host, uploaded once.
    NeuralNetwork(int input_size, int hidden1, int hidden2, int output_size, float lr) : learning_rate(lr) {
        W1 = xavier(size_t(input_size), size_t(hidden1));
        W2 = xavier(size_t(hidden1), size_t(hidden2));
        W3 = xavier(size_t(hidden2), size_t(output_size));
        b1 = Tensor(ShapeTag{}, {size_t(hidden1)}, DType::kFloat, DeviceType::kAMD);
        b2 = Tensor(ShapeTag{}, {size_t(hidden2)}, DType::kFloat, DeviceType::kAMD);
        b3 = Tensor(ShapeTag{}, {size_t(output_size)}, DType::kFloat, DeviceType::kAMD);
    }
    // Given parameter values (host arrays), for tests.
    NeuralNetwork(const float* w1, const float* c1, const float* w2, const float* c2, const float* w3, const float* c3,
                  size_t I, size_t H1, size_t H2, size_t C, float lr)
        : learning_rate(lr) {
        W1 = Tensor::from_host(w1, {I, H1}, DeviceType::kAMD);
        b1 = Tensor::from_host(c1, {H1}, DeviceType::kAMD);
        W2 = Tensor::from_host(w2, {H1, H2}, DeviceType::kAMD);
        b2 = Tensor::from_host(c2, {H2}, DeviceType::kAMD);
        W3 = Tensor::from_host(w3, {H2, C}, DeviceType::kAMD);
        b3 = Tensor::from_host(c3, {C}, DeviceType::kAMD);
    }

    // true: each layer is one fused operator (Tensor::linear); same values and gradients, fewer launches
    bool fused_layers = false;
    // with fused_layers: the last layer, its cross entropy (on the class indices themselves, no one-hot
    // matrix) and the gradients that leave them in one pass (Tensor::linear_cross_entropy); values
    // within the MatMul bound of the other forms
    bool fused_head = false;

    Tensor forward(const Tensor& x) {
        if (fused_layers) return x.linear(W1, b1, true).linear(W2, b2, true).linear(W3, b3, false);
        Tensor h1 = (x.matmul(W1) + b1).relu();
        Tensor h2 = (h1.matmul(W2) + b2).relu();
        return h2.matmul(W3) + b3;
    }

    // One step on a batch; returns the (sum-reduced) loss.  Needs an active AutoDiffContext.
    float train_step(const Tensor& x, const Tensor& y) { return train_step_on_device(x, y).item<float>(); }

    // The same step without reading the loss back: nothing in it makes the host wait for the
    // device, so it can be recorded into a DeviceGraph.  (The reference reads the loss between
    // forward and backward, mnist/mnist.cpp:80-81; the value is the same wherever it is read.)
    Tensor train_step_on_device(const Tensor& x, const Tensor& y) {
        AutoDiff* ctx = AutoDiffContext::current();
        Tensor* params[6] = {&W1, &b1, &W2, &b2, &W3, &b3};
        if (ctx)
            for (Tensor* p : params) ctx->make_leaf(*p, true);
        for (Tensor* p : params) p->requires_grad(true);
        if (ctx)
            for (Tensor* p : params) ctx->zero_grad(*p);
        Tensor loss;
        if (fused_layers && fused_head) {
            loss = x.linear(W1, b1, true).linear(W2, b2, true).linear_cross_entropy(W3, b3, y);
        } else {
            Tensor logits = forward(x);
            Tensor y_one_hot = ctorch_amd_host::onehot(y, logits.sizes()[1]);
            loss = logits.cross_entropy(y_one_hot);
        }
        backward(loss);
        update_parameters();
        return loss;
    }

    void update_parameters() {
        Tensor* params[6] = {&W1, &b1, &W2, &b2, &W3, &b3};
        AutoDiff* ctx = AutoDiffContext::current();
        if (fused_layers && ctx) {                       // one launch for the six tensors
            std::vector<Tensor*> ps(params, params + 6);
            std::vector<Tensor> gs;
            for (Tensor* p : params) gs.push_back(ctx->stored_grad(*p));
            ctorch_amd_host::sgd_step_all(ps, gs, learning_rate);
            return;
        }
        for (Tensor* p : params) {
            Tensor g = grad(*p);
            ctorch_amd_host::sgd_step(*p, g, learning_rate);
        }
    }

    // Row softmax of the logits (mnist/mnist.cpp:95-130).
    Tensor predict(const Tensor& x) { return forward(x).softmax(1); }

   private:
    static Tensor xavier(size_t fan_in, size_t fan_out) {
        std::vector<float> w(fan_in * fan_out);
        float scale = std::sqrt(1.0f / fan_in);
        for (float& v : w) {
            float r = (2.0f * rand() / static_cast<float>(RAND_MAX)) - 1.0f;
            v = r * scale;
        }
        return Tensor::from_host(w.data(), {fan_in, fan_out}, DeviceType::kAMD);
    }
};

// Fraction of rows whose first maximum is at the label (mnist/mnist.cpp:134-156).
inline float calculate_accuracy(const Tensor& y_pred, const Tensor& y_true) {
    int total = int(y_true.shape()[0]);
    return static_cast<float>(ctorch_amd_host::count_correct(y_pred, y_true)) / total;
}

// Rows [batch_idx*batch_size, ...) of the data set as views (mnist/mnist.cpp:159-182 copies them).
inline void get_batch(const Tensor& images, const Tensor& labels, int batch_size, int batch_idx, Tensor& batch_images,
                      Tensor& batch_labels) {
    size_t start = size_t(batch_idx) * size_t(batch_size);
    size_t end = start + size_t(batch_size);
    if (end > images.shape()[0]) end = images.shape()[0];
    batch_images = Tensor::view_rows(images, start, end - start);
    batch_labels = Tensor::view_rows(labels, start, end - start);
}

#endif
