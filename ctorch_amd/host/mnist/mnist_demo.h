// The batch loop of the reference's MNIST demo (main() of mnist/mnist.cpp:220-283) as a function:
// load the four IDX files from a directory, train, evaluate.  mnist.cpp prints what this returns;
// tests call it in process.
#ifndef CTORCH_AMD_HOST_MNIST_DEMO_H
#define CTORCH_AMD_HOST_MNIST_DEMO_H

#include <chrono>
#include <string>
#include <vector>

#include "DeviceGraph.h"
#include "mnist_loader.h"
#include "mnist_model.h"

struct MnistDemoOptions {
    std::string dir = ".";
    int epochs = 5, batch_size = 128, hidden1 = 128, hidden2 = 64;
    float learning_rate = 0.01f;
    unsigned seed = 42;
    // true: the reference's tape (row-0 bias gradients, leaf values frozen at first sight, tape
    // never cleared); false: column sums, live leaves, tape cleared after every step
    bool reference_tape = false;
    // record one training step into a DeviceGraph and replay it per batch (one launch per step
    // instead of ~50); needs reference_tape == false (a frozen leaf copy would be re-made by
    // every replay)
    bool use_graph = false;
    // each layer as one fused operator (Tensor::linear) and the optimiser update as one launch
    bool fused_layers = false;
    // with fused_layers: the last layer and its loss as the one-pass head (Tensor::linear_cross_entropy)
    bool fused_head = false;
    // true (the default): the batch losses of an epoch are added up on the device, in the order and
    // precision the reference adds them on the host (fp32, batch after batch), and read once per epoch -
    // no step makes the host wait, so the host runs ahead and the device never idles between steps.
    // false: every step reads its loss, as the reference's loop does for its progress line
    // (mnist/mnist.cpp:253-260).
    bool loss_on_device = true;
};

struct MnistDemoResult {
    size_t train_images = 0, test_images = 0, pixels = 0;
    int num_batches = 0;
    std::vector<float> epoch_loss;       // mean of the batch losses of each epoch, accumulated in fp32
    float train_accuracy = 0, test_accuracy = 0;
    double train_seconds = 0;
};

inline MnistDemoResult run_mnist_demo(const MnistDemoOptions& opt) {
    MnistDemoResult res;
    // The device first: bringing the GPU runtime up draws from the C library's rand(), and the weights
    // below must be the ones the reference draws after srand(seed) (mnist/mnist.cpp:24-29, :225) - without
    // this the first demo of a process trained from other weights than every later one.
    ctorch_amd_host::init_device();
    srand(opt.seed);
    MNISTLoader loader(opt.dir);
    Tensor train_images, train_labels, test_images, test_labels;
    loader.load_training_data(train_images, train_labels);
    loader.load_test_data(test_images, test_labels);
    res.train_images = train_images.shape()[0];
    res.test_images = test_images.shape()[0];
    res.pixels = train_images.shape()[1];
    NeuralNetwork model(int(res.pixels), opt.hidden1, opt.hidden2, 10, opt.learning_rate);
    model.fused_layers = opt.fused_layers;
    model.fused_head = opt.fused_head;
    res.num_batches = int(res.train_images) / opt.batch_size;

    AutoDiff autodiff;
    if (opt.reference_tape) {
        autodiff.set_broadcast_grad(BroadcastGrad::kReferenceRow0);
        autodiff.set_leaf_values(LeafValues::kReferenceFirstSeen);
    }
    AutoDiffContext::Guard guard(&autodiff);
    if (opt.use_graph && opt.reference_tape)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::TENSOR_STATE, "the recorded step needs live leaves");
    DeviceGraph step;
    Tensor staged_images, staged_labels, staged_loss;
    if (opt.use_graph && res.num_batches > 0) {
        // the recorded step reads its batch from two fixed tensors; each batch is copied into them
        staged_images = Tensor(ShapeTag{}, {size_t(opt.batch_size), res.pixels}, DType::kFloat, DeviceType::kAMD, false);
        staged_labels = Tensor(ShapeTag{}, {size_t(opt.batch_size)}, DType::kFloat, DeviceType::kAMD, false);
    }
    auto t0 = std::chrono::steady_clock::now();
    for (int epoch = 0; epoch < opt.epochs; ++epoch) {
        float epoch_loss = 0.0f;
        Tensor epoch_sum;                   // with loss_on_device: epoch_loss as a device scalar
        if (opt.loss_on_device && !opt.use_graph) epoch_sum = ctorch_amd_host::filled({}, 0.0f, DeviceType::kAMD);
        for (int batch = 0; batch < res.num_batches; ++batch) {
            Tensor batch_images, batch_labels;
            get_batch(train_images, train_labels, opt.batch_size, batch, batch_images, batch_labels);
            if (opt.use_graph) {
                ctorch_amd_host::copy_into(staged_images, batch_images);
                ctorch_amd_host::copy_into(staged_labels, batch_labels);
                if (!step.recorded()) {
                    step.record([&] { staged_loss = model.train_step_on_device(staged_images, staged_labels); });
                    autodiff.clear_graph();
                }
                step.replay();
                epoch_loss += staged_loss.item<float>();
                continue;
            }
            if (opt.loss_on_device) {
                Tensor loss = model.train_step_on_device(batch_images, batch_labels);
                ctorch_amd_host::accumulate(epoch_sum, loss);       // epoch_sum = epoch_sum + loss, the same fp32 addition
            } else {
                epoch_loss += model.train_step(batch_images, batch_labels);
            }
            if (!opt.reference_tape) autodiff.clear_graph();
        }
        if (opt.loss_on_device && !opt.use_graph && res.num_batches > 0) epoch_loss = epoch_sum.item<float>();
        epoch_loss /= static_cast<float>(res.num_batches);
        res.epoch_loss.push_back(epoch_loss);
    }
    res.train_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    res.test_accuracy = calculate_accuracy(model.predict(test_images), test_labels);
    res.train_accuracy = calculate_accuracy(model.predict(train_images), train_labels);
    return res;
}

#endif
