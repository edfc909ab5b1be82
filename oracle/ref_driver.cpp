// TEST INFRASTRUCTURE ONLY.  A plain-C doorway into the real reference library so that the
// CPU restatement in ctorch_oracle.c can be compared with it bit for bit, and so that golden
// vectors can be written from it.  It is compiled (by oracle/Makefile) together with the
// reference's own sources, which are read where they lie and are never copied here; the
// result goes to oracle/_ref/.  Nothing in the product links, loads or calls this file.
//
// Every entry point takes flat fp32 arrays plus shapes, builds reference `Tensor`s, runs the
// reference's own operator / autograd code and copies the result back.  A negative return
// value means the reference threw (-1) or returned an empty tensor (-2).
#include "Tensor.h"
#include "AutoDiff.h"
#include "Ctorch_Error.h"
#include "Ctorch_Scheduler.h"

#include <cstring>
#include <vector>

namespace {

std::vector<size_t> shape_of(const long* dims, int nd) {
    std::vector<size_t> s;
    for (int i = 0; i < nd; ++i) s.push_back(static_cast<size_t>(dims[i]));
    return s;
}

Tensor make(const float* src, const long* dims, int nd) {
    if (nd == 0) return Tensor(src[0]);
    Tensor t(ShapeTag{}, shape_of(dims, nd), DType::kFloat, DeviceType::kCPU);
    if (t.numel()) std::memcpy(t.data<float>(), src, t.numel() * sizeof(float));
    return t;
}

long emit(const Tensor& t, float* dst) {
    if (t.numel() == 0) return -2;
    const float* src = t.data<float>();
    if (src == nullptr) return -2;  // the reference's "empty Tensor()" error return
    std::memcpy(dst, src, t.numel() * sizeof(float));
    return static_cast<long>(t.numel());
}

// op codes shared with the Python side (tests/support.py)
enum Code {
    kAdd = 0, kSub = 1, kMul = 2, kDiv = 3, kMatMul = 4, kDot = 5, kMSE = 6, kMAE = 7, kCE = 8,
    kNeg = 20, kReLU = 21, kSin = 22, kCos = 23, kTanh = 24, kSigmoid = 25, kSoftmaxKernel = 26
};

Tensor run_binary(int code, const Tensor& a, const Tensor& b) {
    switch (code) {
        case kAdd: return a + b;
        case kSub: return a - b;
        case kMul: return a * b;
        case kDiv: return a / b;
        case kMatMul: return a.matmul(b);
        case kDot: return a.dot(b);
        case kMSE: return a.mse_loss(b);
        case kMAE: return a.mae_loss(b);
        case kCE: return a.cross_entropy(b);
    }
    throw std::runtime_error("bad binary code");
}

Tensor run_unary(int code, const Tensor& a) {
    switch (code) {
        case kNeg: return -a;
        case kReLU: return a.relu();
        case kSin: return a.sin();
        case kCos: return a.cos();
        case kTanh: return a.tanh();
        case kSigmoid: return a.sigmoid();
        case kSoftmaxKernel: return Softmax_BASIC_kernel(a);
    }
    throw std::runtime_error("bad unary code");
}

}  // namespace

extern "C" {

void ref_quiet() { Ctorch_Error::setPrintLevel(PrintLevel::MINIUM); }

long ref_binary(int code, const float* a, const long* ad, int an, const float* b, const long* bd,
                int bn, float* out) {
    try {
        Tensor ta = make(a, ad, an), tb = make(b, bd, bn);
        return emit(run_binary(code, ta, tb), out);
    } catch (const std::exception&) {
        return -1;
    }
}

long ref_unary(int code, const float* a, const long* ad, int an, float* out) {
    try {
        Tensor ta = make(a, ad, an);
        return emit(run_unary(code, ta), out);
    } catch (const std::exception&) {
        return -1;
    }
}

// tensor (op) host scalar: which = 0 '+', 1 '*', 2 '/'
long ref_scalar(int which, const float* a, const long* ad, int an, float s, float* out) {
    try {
        Tensor ta = make(a, ad, an);
        Tensor r = which == 0 ? ta + s : which == 1 ? ta * s : ta / s;
        return emit(r, out);
    } catch (const std::exception&) {
        return -1;
    }
}

long ref_sum(const float* a, const long* ad, int an, float* out) {
    try {
        return emit(make(a, ad, an).sum(), out);
    } catch (const std::exception&) {
        return -1;
    }
}

long ref_softmax(const float* a, const long* ad, int an, int dim, float* out) {
    try {
        return emit(make(a, ad, an).softmax(dim), out);
    } catch (const std::exception&) {
        return -1;
    }
}

// Tensors that are not fp32.  The fp32 input goes through the reference's Tensor::to(dtype)
// (dtype in the order of enum DType), then through `n_steps` operations in order, step k being
// whats[k] with scalars[k]: 0 '+ s', 1 '* s', 2 '/ s', 3 zero(), 4 ones(), 5 softmax(dim = (int)s).
// The result's bytes are copied to `out`; returns its element count.
long ref_typed(const float* a, const long* ad, int an, int dtype, const int* whats, const float* scalars, int n_steps,
               void* out) {
    try {
        Tensor t = make(a, ad, an).to(static_cast<DType>(dtype));
        for (int k = 0; k < n_steps; ++k) {
            const float s = scalars[k];
            switch (whats[k]) {
                case 0: t = t + s; break;
                case 1: t = t * s; break;
                case 2: t = t / s; break;
                case 3: t.zero(); break;
                case 4: t.ones(); break;
                case 5: t = t.softmax(static_cast<int>(s)); break;
                default: return -3;
            }
        }
        const size_t n = t.numel();
        switch (t.dtype()) {
            case DType::kFloat: std::memcpy(out, t.data<float>(), n * sizeof(float)); break;
            case DType::kDouble: std::memcpy(out, t.data<double>(), n * sizeof(double)); break;
            case DType::kInt: std::memcpy(out, t.data<int32_t>(), n * sizeof(int32_t)); break;
            case DType::kLong: std::memcpy(out, t.data<int64_t>(), n * sizeof(int64_t)); break;
            case DType::kBool: std::memcpy(out, t.storage().data<bool>(), n * sizeof(bool)); break;   // Tensor::data<bool> is not instantiated
        }
        return static_cast<long>(n);
    } catch (const std::exception&) {
        return -1;
    }
}

// The tape through scalar operators on a tensor that is not fp32: x = to(dtype) of the input,
// y = x through the steps (0 '+ s', 1 '* s', 2 '/ s'), backward(y), grad(x).  The gradient's
// dtype code goes to *grad_dtype and its bytes to grad_out; returns its element count.
long ref_typed_grad(const float* a, const long* ad, int an, int dtype, const int* whats, const float* scalars, int n_steps,
                    void* grad_out, int* grad_dtype) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor x = make(a, ad, an).to(static_cast<DType>(dtype));
        x.requires_grad(true);
        Tensor y = whats[0] == 0 ? x + scalars[0] : whats[0] == 1 ? x * scalars[0] : x / scalars[0];
        for (int k = 1; k < n_steps; ++k) y = whats[k] == 0 ? y + scalars[k] : whats[k] == 1 ? y * scalars[k] : y / scalars[k];
        backward(y);
        Tensor g = grad(x);
        *grad_dtype = static_cast<int>(g.dtype());
        const size_t n = g.numel();
        switch (g.dtype()) {
            case DType::kFloat: std::memcpy(grad_out, g.data<float>(), n * sizeof(float)); break;
            case DType::kDouble: std::memcpy(grad_out, g.data<double>(), n * sizeof(double)); break;
            case DType::kInt: std::memcpy(grad_out, g.data<int32_t>(), n * sizeof(int32_t)); break;
            case DType::kLong: std::memcpy(grad_out, g.data<int64_t>(), n * sizeof(int64_t)); break;
            default: return -3;
        }
        return static_cast<long>(n);
    } catch (const std::exception&) {
        return -1;
    }
}

// C = op(A) * op(B) with op = the reference's t() (deep copy + stride swap) when the flag is set.
// A is stored [am, ak] row-major; ta != 0 multiplies by its transpose, likewise B.
long ref_matmul_t(const float* a, long ar, long ac, int ta, const float* b, long br, long bc, int tb,
                  float* out) {
    try {
        long ad[2] = {ar, ac}, bd[2] = {br, bc};
        Tensor A = make(a, ad, 2), B = make(b, bd, 2);
        Tensor At = ta ? A.t() : A, Bt = tb ? B.t() : B;
        return emit(At.matmul(Bt), out);
    } catch (const std::exception&) {
        return -1;
    }
}

// check_and_adjust_grad_shape (src/AutoDiff.cpp:562-1049, private) through the public
// AutoDiff::backward(root, grad_output), which stores check_and_adjust_grad_shape(grad_output,
// root shape) as the root's gradient (:1124-1126).  The root is a leaf, so nothing else runs.
// The caller must only pass shape pairs for which the reference stays inside the gradient's buffer.
long ref_adjust_grad_shape(const float* g, const long* gd, int gn, const long* td, int tn, float* out) {
    try {
        AutoDiff ctx;
        Tensor tg = make(g, gd, gn);
        Tensor root;
        {
            AutoDiffContext::Guard guard(&ctx);
            if (tn == 0) root = Tensor(0.0f);
            else root = Tensor(ShapeTag{}, shape_of(td, tn), DType::kFloat, DeviceType::kCPU);
            root.requires_grad(true);
        }
        {
            AutoDiffContext::Guard none(nullptr);
            ctx.backward(root, tg);
        }
        AutoDiffContext::Guard guard(&ctx);
        return emit(grad(root), out);
    } catch (const std::exception&) {
        return -1;
    }
}

// d/dx of  sum( f(x) * w )  through the reference's tape: the upstream gradient of f is w.
long ref_grad_unary(int code, const float* x, const long* xd, int xn, const float* w, float* dx) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor tx = make(x, xd, xn), tw = make(w, xd, xn);
        tx.requires_grad(true);
        Tensor y = run_unary(code, tx);
        Tensor z = y * tw;
        Tensor s = z.sum();
        backward(s);
        return emit(grad(tx), dx);
    } catch (const std::exception&) {
        return -1;
    }
}

long ref_grad_softmax(const float* x, const long* xd, int xn, int dim, const float* w, float* dx) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor tx = make(x, xd, xn), tw = make(w, xd, xn);
        tx.requires_grad(true);
        Tensor y = tx.softmax(dim);
        Tensor z = y * tw;
        Tensor s = z.sum();
        backward(s);
        return emit(grad(tx), dx);
    } catch (const std::exception&) {
        return -1;
    }
}

// d/da, d/db of sum( (a op b) * w ); w has the result's shape (wd, wn).
long ref_grad_binary(int code, const float* a, const long* ad, int an, const float* b,
                     const long* bd, int bn, const float* w, const long* wd, int wn, float* da,
                     float* db) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor ta = make(a, ad, an), tb = make(b, bd, bn), tw = make(w, wd, wn);
        ta.requires_grad(true);
        tb.requires_grad(true);
        Tensor y = run_binary(code, ta, tb);
        Tensor z = y * tw;
        Tensor s = z.sum();
        backward(s);
        long r1 = emit(grad(ta), da);
        long r2 = emit(grad(tb), db);
        return (r1 < 0 || r2 < 0) ? -2 : r1 + r2;
    } catch (const std::exception&) {
        return -1;
    }
}

// d/dpred of  loss(pred, target) * scale   (loss in MSE / MAE / CE); the upstream gradient of the
// loss node is then the 0-D value `scale`.
long ref_grad_loss(int code, const float* p, const long* pd, int pn, const float* t, const long* td,
                   int tn, float scale, float* loss_out, float* dp) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        Tensor tp = make(p, pd, pn), tt = make(t, td, tn);
        tp.requires_grad(true);
        Tensor l = run_binary(code, tp, tt);
        if (l.numel() == 0) return -2;
        loss_out[0] = l.item<float>();
        Tensor root = l * scale;
        backward(root);
        return emit(grad(tp), dp);
    } catch (const std::exception&) {
        return -1;
    }
}

// Elementwise chain: c = a*b + 5, d = relu(c), s = d.sum(), s.backward().
long ref_chain(const float* a, const float* b, long n, float* s_out, float* ga, float* gb) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        long d1[1] = {n};
        Tensor ta = make(a, d1, 1), tb = make(b, d1, 1);
        ta.requires_grad(true);
        tb.requires_grad(true);
        Tensor c = ta * tb + 5.0f;
        Tensor d = c.relu();
        Tensor s = d.sum();
        s_out[0] = s.item<float>();
        s.backward();
        emit(grad(ta), ga);
        emit(grad(tb), gb);
        return n;
    } catch (const std::exception&) {
        return -1;
    }
}

// One-hidden-layer MLP step: logits = relu(x*W1 + b1)*W2 + b2, loss = CE_sum(logits, onehot),
// backward to W1, b1, W2, b2.  `onehot` is [B, C].
long ref_mlp_step(const float* x, long B, long I, const float* W1, const float* b1, long H,
                  const float* W2, const float* b2, long C, const float* onehot, float* loss_out,
                  float* logits_out, float* gW1, float* gb1, float* gW2, float* gb2) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        long xd[2] = {B, I}, w1d[2] = {I, H}, b1d[1] = {H}, w2d[2] = {H, C}, b2d[1] = {C},
             yd[2] = {B, C};
        Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1),
               tW2 = make(W2, w2d, 2), tb2 = make(b2, b2d, 1), ty = make(onehot, yd, 2);
        tW1.requires_grad(true);
        tb1.requires_grad(true);
        tW2.requires_grad(true);
        tb2.requires_grad(true);
        Tensor h = (tx.matmul(tW1) + tb1).relu();
        Tensor logits = h.matmul(tW2) + tb2;
        Tensor loss = logits.cross_entropy(ty);
        loss_out[0] = loss.item<float>();
        emit(logits, logits_out);
        backward(loss);
        emit(grad(tW1), gW1);
        emit(grad(tb1), gb1);
        emit(grad(tW2), gW2);
        emit(grad(tb2), gb2);
        return B;
    } catch (const std::exception&) {
        return -1;
    }
}

// Broadcast expression with the row vector materialised by hand (the reference's Div needs equal
// shapes): Y = sigmoid(X / R) - tanh(X) * sin(X) + cos(-X); L = mse(Y,T) + mae(Y,T); one backward.
long ref_expr(const float* X, const float* R, const float* T, long rows, long cols, float* y_out,
              float* mse_out, float* mae_out, float* gX, float* gR) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        long d[2] = {rows, cols};
        Tensor tX = make(X, d, 2), tR = make(R, d, 2), tT = make(T, d, 2);
        tX.requires_grad(true);
        tR.requires_grad(true);
        Tensor q = tX / tR;
        Tensor s1 = q.sigmoid();
        Tensor th = tX.tanh();
        Tensor sn = tX.sin();
        Tensor m = th * sn;
        Tensor d1 = s1 - m;
        Tensor ng = -tX;
        Tensor cs = ng.cos();
        Tensor Y = d1 + cs;
        Tensor l1 = Y.mse_loss(tT);
        Tensor l2 = Y.mae_loss(tT);
        Tensor L = l1 + l2;
        emit(Y, y_out);
        mse_out[0] = l1.item<float>();
        mae_out[0] = l2.item<float>();
        backward(L);
        emit(grad(tX), gX);
        emit(grad(tR), gR);
        return rows * cols;
    } catch (const std::exception&) {
        return -1;
    }
}

// A small straight-line program over tensors, for differential tests of the tape.  Values 0 ..
// n_in-1 are the inputs (kinds[i] = 0: [rows, cols], 1: row vector [cols]; all require gradients),
// each op (code, a, b) appends one value: codes 0-3 Add/Sub/Mul/Div of values a and b (same kind,
// or Add of a full tensor and a row vector), 20-25 the unary operators of value a, 30/31/32
// value a (+, *, /) the scalar 0.5 + 0.25 * b.  The last value must be a full tensor: it is
// copied to y_out, L = sum(last * w) goes to l_out, and after backward(L) the gradients of the
// inputs are written to grads_out one after the other.
long ref_program(const float* inputs, const int* kinds, int n_in, const int* ops, int n_ops, const float* w,
                 long rows, long cols, float* y_out, float* l_out, float* grads_out) {
    try {
        AutoDiff ctx;
        AutoDiffContext::Guard guard(&ctx);
        long full[2] = {rows, cols}, vec[1] = {cols};
        std::vector<Tensor> v;
        v.reserve(size_t(n_in + n_ops));
        const float* src = inputs;
        for (int i = 0; i < n_in; ++i) {
            v.push_back(kinds[i] ? make(src, vec, 1) : make(src, full, 2));
            src += kinds[i] ? cols : rows * cols;
        }
        for (int i = 0; i < n_in; ++i) v[size_t(i)].requires_grad(true);
        for (int k = 0; k < n_ops; ++k) {
            const int code = ops[3 * k], a = ops[3 * k + 1], b = ops[3 * k + 2];
            if (code < 20) v.push_back(run_binary(code, v[size_t(a)], v[size_t(b)]));
            else if (code < 30) v.push_back(run_unary(code, v[size_t(a)]));
            else {
                const float s = 0.5f + 0.25f * float(b);
                v.push_back(code == 30 ? v[size_t(a)] + s : code == 31 ? v[size_t(a)] * s : v[size_t(a)] / s);
            }
        }
        Tensor tw = make(w, full, 2);
        Tensor z = v.back() * tw;
        Tensor L = z.sum();
        if (emit(v.back(), y_out) < 0) return -2;
        l_out[0] = L.item<float>();
        backward(L);
        float* dst = grads_out;
        for (int i = 0; i < n_in; ++i) {
            long got = emit(grad(v[size_t(i)]), dst);
            if (got < 0) return -2;
            dst += got;
        }
        return long(dst - grads_out);
    } catch (const std::exception&) {
        return -1;
    }
}

}  // extern "C"
