// The fused forms against the operator-by-operator forms they stand for, bit for bit: Tensor::linear
// against matmul / + / relu (the layer of the reference's mnist/mnist.cpp:39-41), Expr against the
// Tensor operators (the chains of the reference's src/tests/test_tensor_grad.cpp:152-224 and
// test_activation_loss.cpp), on values, gradients, shapes that cannot be fused, and errors.
#include <cstring>
#include <functional>

#include "AutoDiff.h"
#include "Ctorch_Error.h"
#include "Expr.h"
#include "check.h"
#include "ctorch_amd.h"

static bool same_bits(const Tensor& a, const Tensor& b) {
    std::vector<float> x = a.to_vector(), y = b.to_vector();
    return a.sizes() == b.sizes() && x.size() == y.size() && std::memcmp(x.data(), y.data(), x.size() * sizeof(float)) == 0;
}

static std::vector<float> ramp(size_t n, float scale, float shift) {
    std::vector<float> v(n);
    for (size_t i = 0; i < n; ++i) v[i] = std::sin(float(i) * 0.37f + shift) * scale;
    return v;
}

// runs `body` (which returns the result to differentiate) under a fresh tape and returns
// {result, gradients of the given inputs}
static std::vector<Tensor> run(const std::function<Tensor()>& body, std::vector<Tensor*> inputs, BroadcastGrad mode) {
    AutoDiff ctx;
    ctx.set_broadcast_grad(mode);
    AutoDiffContext::Guard guard(&ctx);
    for (Tensor* t : inputs) t->requires_grad(true);
    Tensor y = body();
    Tensor w = Tensor::from_host(ramp(y.numel(), 1.0f, 2.0f).data(), y.sizes(), DeviceType::kAMD);
    Tensor L = (y * w).sum();
    backward(L);
    std::vector<Tensor> out{y};
    for (Tensor* t : inputs) out.push_back(grad(*t));
    return out;
}

static void linear_layer() {
    Tensor x = device_tensor({5, 7}, ramp(35, 1.0f, 0.1f));
    Tensor W = device_tensor({7, 4}, ramp(28, 0.5f, 0.7f));
    Tensor b = device_tensor({4}, ramp(4, 0.3f, 1.3f));
    for (BroadcastGrad mode : {BroadcastGrad::kColumnSum, BroadcastGrad::kReferenceRow0})
        for (bool relu : {true, false}) {
            // (no `relu ? z.relu() : z`: that copies z, and a copy is a new tensor that the tape does not know)
            auto plain = run([&] { Tensor z = x.matmul(W) + b; if (relu) return z.relu(); return z; }, {&x, &W, &b}, mode);
            auto fused = run([&] { return x.linear(W, b, relu); }, {&x, &W, &b}, mode);
            static const char* names[4] = {"value", "dx", "dW", "db"};
            for (size_t k = 0; k < plain.size(); ++k) {
                std::string what = std::string(relu ? "linear(W, b, relu) = relu(x.W + b): " : "linear(W, b) = x.W + b: ") + names[k];
                CHECK(same_bits(plain[k], fused[k]), what.c_str());
            }
        }
    bool threw = false;
    try {
        Tensor wrong = device_tensor({5}, ramp(5, 1.0f, 0.0f));
        x.linear(W, wrong, false);
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw, "linear with a bias of the wrong length throws");
}

static void expression_chain() {
    Tensor X = device_tensor({6, 8}, ramp(48, 2.0f, 0.2f));
    Tensor T = device_tensor({6, 8}, ramp(48, 1.0f, 0.9f));
    std::vector<float> rv = ramp(8, 0.5f, 0.4f);
    for (float& v : rv) v = std::fabs(v) + 0.5f;
    Tensor r = device_tensor({8}, rv);
    for (BroadcastGrad mode : {BroadcastGrad::kReferenceRow0, BroadcastGrad::kColumnSum}) {
        auto plain = run([&] { return (X / r).sigmoid() - X.tanh() * X.sin() + (-X).cos() * T + 0.25f; }, {&X, &r, &T}, mode);
        auto fused = run([&] {
            Expr x(X), t(T);
            return (sigmoid(x / Expr(r)) - tanh(x) * sin(x) + cos(-x) * t + 0.25f).eval();
        }, {&X, &r, &T}, mode);
        Expr::ProgramStats st = Expr::last_program_stats();
        CHECK(st.forward_insns > 0 && st.backward_insns > 0, "the chain ran as device programs");
        CHECK(same_bits(plain[0], fused[0]), "fused chain: value");
        CHECK(same_bits(plain[1], fused[1]) && same_bits(plain[3], fused[3]), "fused chain: gradients of the full operands");
        if (mode == BroadcastGrad::kReferenceRow0) CHECK(same_bits(plain[2], fused[2]), "fused chain: row-vector gradient, reference mode");
        else CHECK(all_close(fused[2], plain[2].to_vector(), 1e-5f), "fused chain: row-vector gradient, column sums");
    }
}

// In the library's default mode the fused program evaluates sigmoid / tanh / sin / cos in single
// precision (a few ulp from the operator-by-operator kernels, which return glibc's floats in both
// modes): values and gradients agree to rounding, not to the bit.
static void expression_chain_single_precision() {
    const int before = ctamd_set_math_mode(CTAMD_MATH_FAST);
    Tensor X = device_tensor({6, 8}, ramp(48, 2.0f, 0.2f));
    Tensor T = device_tensor({6, 8}, ramp(48, 1.0f, 0.9f));
    std::vector<float> rv = ramp(8, 0.5f, 0.4f);
    for (float& v : rv) v = std::fabs(v) + 0.5f;
    Tensor r = device_tensor({8}, rv);
    auto plain = run([&] { return (X / r).sigmoid() - X.tanh() * X.sin() + (-X).cos() * T + 0.25f; }, {&X, &r, &T}, BroadcastGrad::kColumnSum);
    auto fused = run([&] {
        Expr x(X), t(T);
        return (sigmoid(x / Expr(r)) - tanh(x) * sin(x) + cos(-x) * t + 0.25f).eval();
    }, {&X, &r, &T}, BroadcastGrad::kColumnSum);
    CHECK(all_close(fused[0], plain[0].to_vector(), 1e-6f), "fused chain, single-precision mode: value");
    CHECK(all_close(fused[1], plain[1].to_vector(), 2e-6f) && all_close(fused[3], plain[3].to_vector(), 1e-6f),
          "fused chain, single-precision mode: gradients of the full operands");
    CHECK(all_close(fused[2], plain[2].to_vector(), 1e-5f), "fused chain, single-precision mode: row-vector gradient");
    ctamd_set_math_mode(before);
}

static void same_operand_twice() {
    // x - x and x / x: the reference's tape counts both visits as the first operand (2g and 2g/x)
    Tensor X = device_tensor({4, 4}, ramp(16, 1.0f, 0.3f));
    std::vector<float> pos = ramp(16, 1.0f, 0.5f);
    for (float& v : pos) v = std::fabs(v) + 1.0f;
    Tensor P = device_tensor({4, 4}, pos);
    auto plain = run([&] { return (X - X) + (P / P) + X * X; }, {&X, &P}, BroadcastGrad::kColumnSum);
    auto fused = run([&] { Expr x(X), p(P); return ((x - x) + (p / p) + x * x).eval(); }, {&X, &P}, BroadcastGrad::kColumnSum);
    CHECK(same_bits(plain[0], fused[0]) && same_bits(plain[1], fused[1]) && same_bits(plain[2], fused[2]),
          "x - x, p / p, x * x: the tape's operand bookkeeping is reproduced");
}

static void one_dimensional_and_small() {
    // long 1-D tensors are full operands; small ones are combined by the Tensor operators at once
    Tensor a = device_tensor({70000}, ramp(70000, 1.0f, 0.0f));
    Tensor b = device_tensor({70000}, ramp(70000, 1.0f, 1.0f));
    auto plain = run([&] { return (a * b + 5.0f).relu(); }, {&a, &b}, BroadcastGrad::kColumnSum);
    auto fused = run([&] { return (Expr(a) * Expr(b) + 5.0f).relu().eval(); }, {&a, &b}, BroadcastGrad::kColumnSum);
    CHECK(Expr::last_program_stats().forward_insns == 6, "relu(a * b + 5): two loads, three operators, one store");
    CHECK(same_bits(plain[0], fused[0]) && same_bits(plain[1], fused[1]) && same_bits(plain[2], fused[2]), "1-D chain: value and gradients");
    Tensor s = device_tensor({8}, ramp(8, 1.0f, 0.0f));
    Tensor t = device_tensor({8}, ramp(8, 1.0f, 1.0f));
    Tensor M = device_tensor({3, 8}, ramp(24, 1.0f, 2.0f));
    auto plain2 = run([&] { return M + (s * t).tanh(); }, {&M, &s, &t}, BroadcastGrad::kColumnSum);
    auto fused2 = run([&] { return (Expr(M) + tanh(Expr(s) * Expr(t))).eval(); }, {&M, &s, &t}, BroadcastGrad::kColumnSum);
    bool same = true;
    for (size_t k = 0; k < plain2.size(); ++k) same = same && same_bits(plain2[k], fused2[k]);
    CHECK(same, "row vector computed from two small vectors, then broadcast");
}

static void host_and_errors() {
    Tensor h1 = Tensor::from_host(ramp(6, 1.0f, 0.0f).data(), {2, 3}, DeviceType::kCPU);
    bool refused = false;
    try {
        Tensor r = (Expr(h1) + Expr(h1)).eval();   // host tensors go to the Tensor operators, which compute on the device only
        (void)r;
    } catch (const std::exception&) {
        refused = true;
    }
    CHECK(refused, "host operands are not silently computed somewhere else");
    Tensor A = device_tensor({2, 3}, ramp(6, 1.0f, 0.0f));
    Tensor B = device_tensor({3, 2}, ramp(6, 1.0f, 0.0f));
    bool threw = false;
    try {
        (Expr(A) + Expr(B)).eval();
    } catch (const std::exception&) {
        threw = true;
    }
    CHECK(threw, "operands of different shapes throw");
    // a zero divisor is refused when the gradient is taken, as by the tape's Div branch
    Tensor Z = device_tensor({2, 3}, {1, 2, 0, 4, 5, 6});
    bool div_threw = false;
    try {
        run([&] { return (Expr(A) / Expr(Z) + 1.0f).eval(); }, {&A, &Z}, BroadcastGrad::kColumnSum);
    } catch (const std::exception&) {
        div_threw = true;
    }
    CHECK(div_threw, "gradient of a division by a tensor with a zero throws");
}

int main() {
    Ctorch_Error::setPrintLevel(PrintLevel::MINIUM);
    ctamd_set_math_mode(CTAMD_MATH_EXACT);   // the bit-for-bit comparisons below hold in this mode
    linear_layer();
    expression_chain();
    expression_chain_single_precision();
    same_operand_twice();
    one_dimensional_and_small();
    host_and_errors();
    std::printf("%d failure(s)\n", g_failures);
    return g_failures;
}
