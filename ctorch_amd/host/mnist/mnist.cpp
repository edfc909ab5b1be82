// The reference's MNIST demo (mnist/mnist.cpp:220-283) on the MI355X: same model, batch loop and
// printed results, data set and parameters resident in HBM.
//
//   mnist.bin [--data DIR] [--epochs N] [--batch N] [--lr X] [--hidden1 N] [--hidden2 N]
//             [--reference-tape | --graph] [--fused | --fused-head] [--loss-each-step]
//
// --graph records one training step into a HIP graph at the first batch and replays it for every
// batch: one launch per step instead of about fifty.
//
// --reference-tape reproduces two properties of the reference's tape that change the numbers:
// bias gradients taken from row 0 of the upstream gradient, and leaf values frozen at their
// first-step copies in backward; without it the tape is cleared after every step, bias gradients
// are column sums and backward reads live weights.
#include <cstdio>
#include <cstdlib>
#include <iomanip>
#include <iostream>
#include <string>

#include "Ctorch_Error.h"
#include "mnist_demo.h"

int main(int argc, char** argv) {
    MnistDemoOptions opt;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto next = [&]() -> const char* { return i + 1 < argc ? argv[++i] : ""; };
        if (a == "--data") opt.dir = next();
        else if (a == "--epochs") opt.epochs = std::atoi(next());
        else if (a == "--batch") opt.batch_size = std::atoi(next());
        else if (a == "--lr") opt.learning_rate = float(std::atof(next()));
        else if (a == "--hidden1") opt.hidden1 = std::atoi(next());
        else if (a == "--hidden2") opt.hidden2 = std::atoi(next());
        else if (a == "--reference-tape") opt.reference_tape = true;
        else if (a == "--graph") opt.use_graph = true;
        else if (a == "--fused") opt.fused_layers = true;
        else if (a == "--fused-head") opt.fused_layers = opt.fused_head = true;
        else if (a == "--loss-each-step") opt.loss_on_device = false;
        else {
            std::fprintf(stderr, "unknown option %s\n", a.c_str());
            return 2;
        }
    }
    try {
        Ctorch_Error::setPrintLevel(PrintLevel::MINIUM);
        std::cout << "net: ->" << opt.hidden1 << "->" << opt.hidden2 << "->10 | epochs:" << opt.epochs
                  << " | batch:" << opt.batch_size << " | lr:" << opt.learning_rate << std::endl;
        MnistDemoResult r = run_mnist_demo(opt);
        std::cout << "MNIST loaded | train:" << r.train_images << " test:" << r.test_images << std::endl;
        for (size_t e = 0; e < r.epoch_loss.size(); ++e)
            std::cout << "Epoch " << (e + 1) << "/" << opt.epochs << " Loss: " << std::fixed << std::setprecision(4)
                      << r.epoch_loss[e] << std::endl;
        std::cout << ">>> train accuracy: " << std::fixed << std::setprecision(2) << (r.train_accuracy * 100) << "%" << std::endl;
        std::cout << ">>> test accuracy: " << std::fixed << std::setprecision(2) << (r.test_accuracy * 100) << "%" << std::endl;
        std::cout << "training: " << std::setprecision(3) << r.train_seconds << " s, " << std::setprecision(1)
                  << (r.train_seconds * 1e6 / (double(opt.epochs) * r.num_batches)) << " us per step" << std::endl;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "error: %s\n", e.what());
        return 1;
    }
    return 0;
}
