// Activations and losses on the device, after the reference's src/tests/test_activation_loss.cpp:
// softmax rows / columns sum to 1 (:57-65, :94-112), d(sum(softmax))/dx ~ 0 (:114-126),
// CE(1-D one-hot) == -log(softmax[true]) (:156-170), dCE/dz == softmax - target (:172-189);
// sigmoid / tanh / relu / MSE / MAE run there without value checks (:44-86, :138-152, :191-272) and
// are given known answers here.
#include "check.h"

static float sum_of(const std::vector<float>& v, size_t begin, size_t step, size_t count) {
    double s = 0;
    for (size_t i = 0; i < count; ++i) s += v[begin + i * step];
    return float(s);
}

static void softmax_checks() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor v = device_tensor({4}, {1.0f, 2.0f, 3.0f, 4.0f});
    std::vector<float> p = v.softmax().to_vector();
    CHECK(std::fabs(sum_of(p, 0, 1, 4) - 1.0f) < 1e-6f && p[3] > p[2] && p[2] > p[1], "1-D softmax sums to 1 and is monotone");
    Tensor m = device_tensor({2, 3}, {1, 2, 3, 1, 5, 2});
    std::vector<float> r = m.softmax(1).to_vector(), c = m.softmax(0).to_vector();
    CHECK(std::fabs(sum_of(r, 0, 1, 3) - 1) < 1e-6f && std::fabs(sum_of(r, 3, 1, 3) - 1) < 1e-6f, "softmax(dim=1): rows sum to 1");
    CHECK(std::fabs(sum_of(c, 0, 3, 2) - 1) < 1e-6f && std::fabs(sum_of(c, 2, 3, 2) - 1) < 1e-6f, "softmax(dim=0): columns sum to 1");
    m.requires_grad(true);
    Tensor y = m.softmax(1);
    Tensor s = y.sum();
    s.backward();
    std::vector<float> g = grad(m).to_vector();
    float worst = 0;
    for (float x : g) worst = std::fmax(worst, std::fabs(x));
    CHECK(worst < 1e-4f, "d(sum(softmax(x)))/dx ~ 0");
}

static void cross_entropy_checks() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor z = device_tensor({4}, {0.5f, 2.0f, -1.0f, 0.1f});
    Tensor t = device_tensor({4}, {0, 1, 0, 0});
    z.requires_grad(true);
    std::vector<float> p = z.softmax().to_vector();
    Tensor loss = z.cross_entropy(t);
    CHECK(std::fabs(loss.item<float>() - (-std::log(p[1]))) < 1e-4f, "CE(one-hot) = -log softmax[true]");
    backward(loss);
    std::vector<float> want = {p[0], p[1] - 1.0f, p[2], p[3]};
    CHECK(all_close(grad(z), want, 1e-4f), "dCE/dz = softmax - target");
    // batch with class indices: the loss is the SUM over the rows
    Tensor zz = device_tensor({2, 3}, {1, 2, 3, 1, 2, 3});
    Tensor idx = device_tensor({2}, {2, 0});
    float lse = std::log(std::exp(1.0f) + std::exp(2.0f) + std::exp(3.0f));
    CHECK(std::fabs(zz.cross_entropy(idx).item<float>() - ((lse - 3) + (lse - 1))) < 1e-4f, "CE with class indices sums over rows");
    Tensor bad = device_tensor({2}, {2, 3});
    CHECK(zz.cross_entropy(bad).is_cleared(), "out-of-range class index returns an empty Tensor");
}

static void activations_and_losses() {
    AutoDiff ctx;
    AutoDiffContext::Guard guard(&ctx);
    Tensor x = device_tensor({3}, {-1.0f, 0.0f, 2.0f});
    CHECK(all_close(x.sigmoid(), {0.26894143f, 0.5f, 0.88079709f}, 1e-6f), "sigmoid values");
    CHECK(all_close(x.tanh(), {-0.76159418f, 0.0f, 0.96402758f}, 1e-6f), "tanh values");
    CHECK(all_close(x.relu(), {0.0f, 0.0f, 2.0f}, 0.0f), "relu values");
    CHECK(all_close(x.sin(), {-0.84147098f, 0.0f, 0.90929743f}, 1e-6f), "sin values");
    CHECK(all_close(x.cos(), {0.54030231f, 1.0f, -0.41614684f}, 1e-6f), "cos values");
    Tensor p = device_tensor({4}, {1, 2, 3, 4}), t = device_tensor({4}, {1, 1, 5, 2});
    p.requires_grad(true);
    Tensor mse = p.mse_loss(t), mae = p.mae_loss(t);
    CHECK(std::fabs(mse.item<float>() - 2.25f) < 1e-6f, "MSE = mean squared difference");
    CHECK(std::fabs(mae.item<float>() - 1.25f) < 1e-6f, "MAE = mean absolute difference");
    Tensor total = mse + mae;
    backward(total);
    // d/dp = 2(p - t)/n + sign(p - t)/n
    CHECK(all_close(grad(p), {0.0f, 0.75f, -1.25f, 1.25f}, 1e-6f), "d(MSE + MAE)/dp");
    Tensor a = device_tensor({2, 2}, {1, 2, 3, 4}), b = device_tensor({2, 2}, {5, 6, 7, 8});
    CHECK(all_close(a.matmul(b), {19, 22, 43, 50}, 0.0f), "matmul values");
    CHECK(all_close(a.t().matmul(b), {26, 30, 38, 44}, 0.0f), "matmul of a transposed view");
    CHECK(std::fabs(a.dot(b).item<float>() - 70.0f) < 1e-6f, "dot value");
    CHECK(std::fabs(a.sum().item<float>() - 10.0f) < 1e-6f, "sum value");
}

int main() {
    Ctorch_Error::setPrintLevel(PrintLevel::MINIUM);
    softmax_checks();
    cross_entropy_checks();
    activations_and_losses();
    std::printf("%d failure(s)\n", g_failures);
    return g_failures;
}
