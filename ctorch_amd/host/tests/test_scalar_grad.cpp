// Scalar autograd on the device, after the reference's src/tests/test.cpp:6-155: gradients of
// a+b, a*b, a-b, -a and a/b on 0-D tensors (1e-6), plus the ReLU gradient that the reference's
// program has but keeps disabled (:157-196).
#include "check.h"

static void add_mul_sub_neg_div() {
    {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor a(2.0f, DeviceType::kAMD), b(3.0f, DeviceType::kAMD);
        a.requires_grad(true);
        b.requires_grad(true);
        Tensor c = a + b;
        backward(c);
        CHECK(std::fabs(grad(a).item<float>() - 1.0f) < 1e-6f && std::fabs(grad(b).item<float>() - 1.0f) < 1e-6f, "d(a+b) = (1, 1)");
    }
    {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor a(2.0f, DeviceType::kAMD), b(3.0f, DeviceType::kAMD);
        a.requires_grad(true);
        b.requires_grad(true);
        Tensor c = a * b;
        backward(c);
        CHECK(std::fabs(grad(a).item<float>() - 3.0f) < 1e-6f && std::fabs(grad(b).item<float>() - 2.0f) < 1e-6f, "d(a*b) = (b, a)");
    }
    {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor a(5.0f, DeviceType::kAMD), b(3.0f, DeviceType::kAMD);
        a.requires_grad(true);
        b.requires_grad(true);
        Tensor c = a - b;
        backward(c);
        CHECK(std::fabs(grad(a).item<float>() - 1.0f) < 1e-6f && std::fabs(grad(b).item<float>() + 1.0f) < 1e-6f, "d(a-b) = (1, -1)");
    }
    {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor a(4.0f, DeviceType::kAMD);
        a.requires_grad(true);
        Tensor c = -a;
        backward(c);
        CHECK(std::fabs(grad(a).item<float>() + 1.0f) < 1e-6f, "d(-a) = -1");
    }
    {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor a(6.0f, DeviceType::kAMD), b(2.0f, DeviceType::kAMD);
        a.requires_grad(true);
        b.requires_grad(true);
        Tensor c = a / b;
        backward(c);
        CHECK(std::fabs(grad(a).item<float>() - 0.5f) < 1e-6f && std::fabs(grad(b).item<float>() + 1.5f) < 1e-6f, "d(a/b) = (1/b, -a/b^2)");
    }
}

static void relu_gradient() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor x = device_tensor({4}, {-1.5f, 0.0f, 2.0f, 3.5f});
    x.requires_grad(true);
    Tensor y = x.relu();
    Tensor s = y.sum();
    s.backward();
    CHECK(all_close(y, {0.0f, 0.0f, 2.0f, 3.5f}, 0.0f), "relu forward");
    CHECK(all_close(grad(x), {0.0f, 0.0f, 1.0f, 1.0f}, 0.0f), "relu gradient is the x > 0 mask");
}

static void errors() {
    bool threw = false;
    try {
        Tensor host_a(1.0f), host_b(2.0f);
        Tensor c = host_a + host_b;   // host tensors have no kernels in this library
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw, "dispatch on a host tensor reports 'no kernel' by throwing");
    threw = false;
    try {
        Tensor d(1.0f, DeviceType::kAMD);
        (void)d.data<float>();
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw, "data<T>() on a device tensor throws");
    threw = false;
    try {
        Tensor d(1.0f, DeviceType::kAMD), h(1.0f);
        Tensor c = d + h;
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw, "operands on different devices throw");
    Tensor h = device_tensor({3}, {1.0f, 2.0f, 3.0f}).cpu();
    CHECK(h.device() == DeviceType::kCPU && h.data<float>()[2] == 3.0f, "explicit transfer back to the host");
}

int main() {
    Ctorch_Error::setPrintLevel(PrintLevel::MINIUM);
    add_mul_sub_neg_div();
    relu_gradient();
    errors();
    std::printf("%d failure(s)\n", g_failures);
    return g_failures;
}
