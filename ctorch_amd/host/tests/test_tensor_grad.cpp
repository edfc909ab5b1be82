// Tensor autograd on the device, after the reference's src/tests/test_tensor_grad.cpp:
// d(2*(a+b)) is all 2 on [2,3] (:7-73); a[2,3] + b[3] with c as root (:76-149) - the reference
// expects db == 1 (row 0 of the upstream gradient), the complete gradient is the column sum 2,
// both modes are checked; z = x*y + x gives dx = y + 1, dy = x (:152-224).
#include "check.h"

static void tensor_gradient() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor a = device_tensor({2, 3}, {0, 1, 2, 3, 4, 5});
    Tensor b = device_tensor({2, 3}, {6, 5, 4, 3, 2, 1});
    a.requires_grad(true);
    b.requires_grad(true);
    Tensor c = a + b;
    Tensor d = c * 2.0f;
    backward(d);
    CHECK(all_equal_to(d, 12.0f, 0.0f), "2*(a+b) forward");
    CHECK(all_equal_to(grad(a), 2.0f, 1e-6f) && all_equal_to(grad(b), 2.0f, 1e-6f), "d(2*(a+b)) = 2 everywhere");
}

static void broadcast_gradient(BroadcastGrad mode, float expected_db, const char* what) {
    AutoDiff ctx;
    ctx.set_broadcast_grad(mode);
    AutoDiffContext::Guard guard(&ctx);
    Tensor a = device_tensor({2, 3}, {0, 1, 2, 3, 4, 5});
    Tensor b = device_tensor({3}, {1, 2, 3});
    a.requires_grad(true);
    b.requires_grad(true);
    Tensor c = a + b;
    backward(c);
    CHECK(all_close(c, {1, 3, 5, 4, 6, 8}, 0.0f), "a[2,3] + b[3] forward");
    CHECK(all_equal_to(grad(a), 1.0f, 1e-6f), "da = 1");
    CHECK(grad(b).numel() == 3 && all_equal_to(grad(b), expected_db, 1e-6f), what);
}

static void product_plus() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor x = device_tensor({2, 2}, {1, 2, 3, 4});
    Tensor y = device_tensor({2, 2}, {5, 6, 7, 8});
    x.requires_grad(true);
    y.requires_grad(true);
    Tensor z = x * y + x;
    backward(z);
    CHECK(all_close(grad(x), {6, 7, 8, 9}, 1e-6f), "d(x*y + x)/dx = y + 1");
    CHECK(all_close(grad(y), {1, 2, 3, 4}, 1e-6f), "d(x*y + x)/dy = x");
}

static void square_counts_both_uses() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor x = device_tensor({3}, {1, -2, 3});
    x.requires_grad(true);
    Tensor y = x * x;
    Tensor s = y.sum();
    s.backward();
    CHECK(all_close(grad(x), {2, -4, 6}, 1e-6f), "d(sum(x*x))/dx = 2x (the operand is visited twice)");
}

int main() {
    Ctorch_Error::setPrintLevel(PrintLevel::MINIUM);
    tensor_gradient();
    broadcast_gradient(BroadcastGrad::kReferenceRow0, 1.0f, "db = 1 in the reference's row-0 mode");
    broadcast_gradient(BroadcastGrad::kColumnSum, 2.0f, "db = 2 as the column sum (default)");
    product_plus();
    square_counts_both_uses();
    std::printf("%d failure(s)\n", g_failures);
    return g_failures;
}
