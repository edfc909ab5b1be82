// C doorway into the host front-end for in-process tests: flat fp32 host arrays in, the operator /
// autograd path through Tensor, Ctorch_Scheduler, the <Op>_AMD_kernel shims and the tape on the
// MI355X, results copied back.  The entry points have the shape of the ones the tests use for the
// reference library, so one test body can drive either.  A negative return value means the call
// threw (-1) or produced an empty tensor (-2).
#include "Tensor.h"
#include "AutoDiff.h"
#include "Expr.h"
#include "Ctorch_Error.h"
#include "Ctorch_Scheduler.h"

#include "ctorch_amd.h"
#include "DeviceGraph.h"
#include "mnist_demo.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

std::vector<size_t> shape_of(const long* dims, int nd) {
    std::vector<size_t> s;
    for (int i = 0; i < nd; ++i) s.push_back(static_cast<size_t>(dims[i]));
    return s;
}

// set: inputs arrive as if a device computation had produced them - the front-end keeps nothing of what
// the upload saw (whether a short vector holds class indices in range), so range checks run on the device
bool g_inputs_unseen = false;
// set: the timed MLP step does not read its loss back, so the host runs ahead of the device and the time per
// step is the larger of the host's time to issue a step and the device's time to run one
bool g_no_loss_read = false;
Tensor make(const float* src, const long* dims, int nd) {
    Tensor t = Tensor::from_host(src, shape_of(dims, nd), DeviceType::kAMD);
    if (g_inputs_unseen) t.forget_known_value();
    return t;
}

long emit(const Tensor& t, float* dst) {
    if (t.numel() == 0 || t.is_cleared()) return -2;   // the "empty Tensor()" error return
    std::vector<float> v = t.to_vector();
    std::memcpy(dst, v.data(), v.size() * sizeof(float));
    return static_cast<long>(v.size());
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

Expr run_binary(int code, const Expr& a, const Expr& b) {
    switch (code) {
        case kAdd: return a + b;
        case kSub: return a - b;
        case kMul: return a * b;
        case kDiv: return a / b;
    }
    throw std::runtime_error("bad binary code");
}

Expr run_unary(int code, const Expr& a) {
    switch (code) {
        case kNeg: return -a;
        case kReLU: return a.relu();
        case kSin: return a.sin();
        case kCos: return a.cos();
        case kTanh: return a.tanh();
        case kSigmoid: return a.sigmoid();
    }
    throw std::runtime_error("bad unary code");
}

Tensor run_unary(int code, const Tensor& a) {
    switch (code) {
        case kNeg: return -a;
        case kReLU: return a.relu();
        case kSin: return a.sin();
        case kCos: return a.cos();
        case kTanh: return a.tanh();
        case kSigmoid: return a.sigmoid();
        case kSoftmaxKernel: return Softmax_AMD_kernel(a);
    }
    throw std::runtime_error("bad unary code");
}

}  // namespace

extern "C" {

void cth_quiet() { Ctorch_Error::setPrintLevel(PrintLevel::MINIUM); }

// 0: gradient of a row-broadcast operand = column sum (default); 1: the reference's row-0 slice.
// Applies to the contexts the entry points below create.
static int g_row0 = 0;
static int g_fused_layers = 0;
static int g_fused_head = 0;
static int g_fused_expr = 0;
extern "C" void cth_set_ce_deferred_label_check(int on) { ctorch_amd_host::set_ce_deferred_label_check(on != 0); }
// the elementwise parts of cth_chain, cth_expr, cth_program and their timed versions are built as
// one fused expression (Expr::eval: one launch forward, one backward) when set
void cth_set_fused_expr(int on) { g_fused_expr = on; }
// class-index cross entropy under a tape: loss and gradient in one pass over the logits (default), or
// a forward pass that leaves row statistics and a streaming backward pass
void cth_set_ce_one_pass(int on) { ctorch_amd_host::set_ce_one_pass(on != 0); }
void cth_set_inputs_unseen(int on) { g_inputs_unseen = on != 0; }
void cth_set_no_loss_read(int on) { g_no_loss_read = on != 0; }
// sizes of the programs the last Expr::eval() compiled: out[0..3] = forward instructions, forward
// slots, backward instructions, backward slots (zeros: evaluated operator by operator)
void cth_last_expr_stats(int* out) {
    Expr::ProgramStats s = Expr::last_program_stats();
    out[0] = s.forward_insns;
    out[1] = s.forward_slots;
    out[2] = s.backward_insns;
    out[3] = s.backward_slots;
}
void cth_set_reference_row0(int on) { g_row0 = on; }
// the MLP entry points below build each layer with Tensor::linear (one fused operator) when set
void cth_set_fused_layers(int on) { g_fused_layers = on; }
// with fused layers: the last layer and its class-index cross entropy as one operator (Tensor::linear_cross_entropy)
void cth_set_fused_head(int on) { g_fused_head = on; }
// the ReLU mask of a fused layer in the product that forms the layer's output gradient (default) or
// as a launch of its own
static int g_fuse_relu_mask = 1;
void cth_set_fuse_relu_mask(int on) { g_fuse_relu_mask = on; }
// the bias gradient of a fused layer with its weight gradient (default) or as launches of its own
static int g_bias_with_weight = 1;
void cth_set_bias_grad_with_weight_grad(int on) { g_bias_with_weight = on; }
static void configure(AutoDiff& ctx) {
    ctx.set_broadcast_grad(g_row0 ? BroadcastGrad::kReferenceRow0 : BroadcastGrad::kColumnSum);
    ctx.set_fuse_relu_mask(g_fuse_relu_mask != 0);
    ctx.set_bias_grad_with_weight_grad(g_bias_with_weight != 0);
}

long cth_binary(int code, const float* a, const long* ad, int an, const float* b, const long* bd,
                int bn, float* out) {
    try {
        Tensor ta = make(a, ad, an), tb = make(b, bd, bn);
        return emit(run_binary(code, ta, tb), out);
    } catch (const std::exception&) {
        return -1;
    }
}

long cth_unary(int code, const float* a, const long* ad, int an, float* out) {
    try {
        Tensor ta = make(a, ad, an);
        return emit(run_unary(code, ta), out);
    } catch (const std::exception&) {
        return -1;
    }
}

// a (cmp) b, or a (cmp) s when b is null; cmp = 0 '>', 1 '<', 2 '==', 3 '>=', 4 '<=', 5 '!='; one byte per element
long cth_compare(int cmp, const float* a, const long* ad, int an, const float* b, const long* bd, int bn, float s,
                 unsigned char* out) {
    try {
        Tensor ta = make(a, ad, an);
        Tensor r;
        if (b) {
            Tensor tb = make(b, bd, bn);
            r = cmp == 0 ? ta > tb : cmp == 1 ? ta < tb : cmp == 2 ? ta == tb : cmp == 3 ? ta >= tb : cmp == 4 ? ta <= tb : ta != tb;
        } else {
            r = cmp == 0 ? ta > s : cmp == 1 ? ta < s : cmp == 2 ? ta == s : cmp == 3 ? ta >= s : cmp == 4 ? ta <= s : ta != s;
        }
        if (r.dtype() != DType::kBool) return -3;
        std::vector<unsigned char> v = r.to_bytes();
        std::memcpy(out, v.data(), v.size());
        return static_cast<long>(v.size());
    } catch (const std::exception&) {
        return -1;
    }
}

// Tensors that are not fp32: the fp32 input through Tensor::to(dtype) (dtype in the order of enum
// DType), then through `n_steps` operations in order, step k being whats[k] with scalars[k]:
// 0 '+ s', 1 '* s', 2 '/ s', 3 zero(), 4 ones(), 5 softmax(dim = (int)s).  The result's bytes are
// copied to `out`; returns its element count.
long cth_typed(const float* a, const long* ad, int an, int dtype, const int* whats, const float* scalars, int n_steps,
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
        std::vector<unsigned char> v = t.to_bytes();
        std::memcpy(out, v.data(), v.size());
        return static_cast<long>(t.numel());
    } catch (const std::exception&) {
        return -1;
    }
}

// The tape through scalar operators on a tensor that is not fp32: backward() of it throws in the
// reference (its float seed meets typed nodes: DATATYPE), and must here; returns -1 then.
long cth_typed_grad(const float* a, const long* ad, int an, int dtype, const int* whats, const float* scalars, int n_steps,
                    void* grad_out, int* grad_dtype) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor x = make(a, ad, an).to(static_cast<DType>(dtype));
        x.requires_grad(true);
        Tensor y = whats[0] == 0 ? x + scalars[0] : whats[0] == 1 ? x * scalars[0] : x / scalars[0];
        for (int k = 1; k < n_steps; ++k) y = whats[k] == 0 ? y + scalars[k] : whats[k] == 1 ? y * scalars[k] : y / scalars[k];
        backward(y);
        Tensor g = grad(x);
        *grad_dtype = static_cast<int>(g.dtype());
        std::vector<unsigned char> v = g.to_bytes();
        std::memcpy(grad_out, v.data(), v.size());
        return static_cast<long>(g.numel());
    } catch (const std::exception&) {
        return -1;
    }
}

// tensor (op) host scalar: which = 0 '+', 1 '*', 2 '/'
long cth_scalar(int which, const float* a, const long* ad, int an, float s, float* out) {
    try {
        Tensor ta = make(a, ad, an);
        Tensor r = which == 0 ? ta + s : which == 1 ? ta * s : ta / s;
        return emit(r, out);
    } catch (const std::exception&) {
        return -1;
    }
}

long cth_sum(const float* a, const long* ad, int an, float* out) {
    try {
        return emit(make(a, ad, an).sum(), out);
    } catch (const std::exception&) {
        return -1;
    }
}

long cth_softmax(const float* a, const long* ad, int an, int dim, float* out) {
    try {
        return emit(make(a, ad, an).softmax(dim), out);
    } catch (const std::exception&) {
        return -1;
    }
}

// C = op(A) * op(B) with op = the reference's t() (deep copy + stride swap) when the flag is set.
// A is stored [am, ak] row-major; ta != 0 multiplies by its transpose, likewise B.
long cth_matmul_t(const float* a, long ar, long ac, int ta, const float* b, long br, long bc, int tb,
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

// d/dx of  sum( f(x) * w )  through the reference's tape: the upstream gradient of f is w.
long cth_grad_unary(int code, const float* x, const long* xd, int xn, const float* w, float* dx) {
    try {
        AutoDiff ctx;
        configure(ctx);
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

long cth_grad_softmax(const float* x, const long* xd, int xn, int dim, const float* w, float* dx) {
    try {
        AutoDiff ctx;
        configure(ctx);
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
long cth_grad_binary(int code, const float* a, const long* ad, int an, const float* b,
                     const long* bd, int bn, const float* w, const long* wd, int wn, float* da,
                     float* db) {
    try {
        AutoDiff ctx;
        configure(ctx);
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

// ---- the methods the reference declares without defining them
namespace {
// 40 abs, 41 exp, 42 log, 43 sqrt, 44 square, 45 tan, 46 leaky_relu(p), 47 a - p,
// 48 op::LReLU through Ctorch_Scheduler::dispatch (the registered kernel, slope 0.01)
Tensor run_declared(int code, const Tensor& a, float p) {
    switch (code) {
        case 40: return a.abs();
        case 41: return a.exp();
        case 42: return a.log();
        case 43: return a.sqrt();
        case 44: return a.square();
        case 45: return a.tan();
        case 46: return a.leaky_relu(p);
        case 47: return a - p;
        case 48: return Ctorch_Scheduler::getInstance().dispatch(a, op::LReLU);
    }
    throw std::runtime_error("bad declared-unary code");
}
// kind 0 sum, 1 mean, 2 max, 3 min, 4 var, 5 std; no dims and no keepdim: the method without arguments
// (sum() is the reference's own full sum); one dim: the (int, bool) overload; ddof < 0: the method's default
Tensor run_reduce(int kind, const Tensor& a, const int* dims, int n_dims, bool keepdim, int ddof) {
    std::vector<int> ds(dims, dims + n_dims);
    if (kind == 4 && ddof >= 0) return a.var_of(ds, keepdim, ddof);
    if (kind == 5 && ddof >= 0) return a.std_of(ds, keepdim, ddof);
    if (n_dims == 0 && !keepdim) {
        switch (kind) {
            case 0: return a.sum();
            case 1: return a.mean();
            case 2: return a.max();
            case 3: return a.min();
            case 4: return a.var();
            case 5: return a.std();
        }
    }
    if (n_dims == 1) {
        switch (kind) {
            case 0: return a.sum(ds[0], keepdim);
            case 1: return a.mean(ds[0], keepdim);
            case 2: return a.max(ds[0], keepdim);
            case 3: return a.min(ds[0], keepdim);
            case 4: return a.var(ds[0], keepdim);
            case 5: return a.std(ds[0], keepdim);
        }
    }
    switch (kind) {
        case 0: return a.sum(ds, keepdim);
        case 1: return a.mean(ds, keepdim);
        case 2: return a.max(ds, keepdim);
        case 3: return a.min(ds, keepdim);
        case 4: return a.var(ds, keepdim);
        case 5: return a.std(ds, keepdim);
    }
    throw std::runtime_error("bad reduction kind");
}
}  // namespace

long cth_declared_unary(int code, const float* a, const long* ad, int an, float p, float* out) {
    try {
        Tensor ta = make(a, ad, an);
        return emit(run_declared(code, ta, p), out);
    } catch (const std::exception&) {
        return -1;
    }
}
// d/dx of sum( f(x) * w )
long cth_grad_declared_unary(int code, const float* x, const long* xd, int xn, float p, const float* w, float* dx) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor tx = make(x, xd, xn), tw = make(w, xd, xn);
        tx.requires_grad(true);
        Tensor y = run_declared(code, tx, p);
        if (code == 48) return -3;              // the bare dispatch is not taped
        Tensor z = y * tw;
        Tensor s = z.sum();
        backward(s);
        return emit(grad(tx), dx);
    } catch (const std::exception&) {
        return -1;
    }
}
// out_dims / out_rank: the result's shape
long cth_reduce(int kind, const float* a, const long* ad, int an, const int* dims, int n_dims, int keepdim, int ddof,
                float* out, long* out_dims, int* out_rank) {
    try {
        Tensor ta = make(a, ad, an);
        Tensor r = run_reduce(kind, ta, dims, n_dims, keepdim != 0, ddof);
        *out_rank = int(r.dim());
        for (size_t i = 0; i < r.dim(); ++i) out_dims[i] = long(r.sizes()[i]);
        return emit(r, out);
    } catch (const std::exception&) {
        return -1;
    }
}
// d/dx of sum( reduce(x) * w ), w of the result's shape
long cth_grad_reduce(int kind, const float* x, const long* xd, int xn, const int* dims, int n_dims, int keepdim, int ddof,
                     const float* w, float* dx) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor tx = make(x, xd, xn);
        tx.requires_grad(true);
        Tensor y = run_reduce(kind, tx, dims, n_dims, keepdim != 0, ddof);
        std::vector<long> yd(y.sizes().begin(), y.sizes().end());
        Tensor tw = make(w, yd.data(), int(yd.size()));
        Tensor z = y * tw;
        Tensor s = z.sum();
        backward(s);
        return emit(grad(tx), dx);
    } catch (const std::exception&) {
        return -1;
    }
}
long cth_log_softmax(const float* a, const long* ad, int an, int dim, float* out) {
    try {
        return emit(make(a, ad, an).log_softmax(dim), out);
    } catch (const std::exception&) {
        return -1;
    }
}
long cth_grad_log_softmax(const float* x, const long* xd, int xn, int dim, const float* w, float* dx) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor tx = make(x, xd, xn), tw = make(w, xd, xn);
        tx.requires_grad(true);
        Tensor y = tx.log_softmax(dim);
        Tensor z = y * tw;
        Tensor s = z.sum();
        backward(s);
        return emit(grad(tx), dx);
    } catch (const std::exception&) {
        return -1;
    }
}
// The gradient a root of shape td ends up with after backward(root, grad_output = g): the tape's
// gradient shape adjustment (the reference's check_and_adjust_grad_shape, src/AutoDiff.cpp:562-1049),
// in the mode cth_set_reference_row0 selected.  The root is a leaf, so nothing else runs.
long cth_adjust_grad_shape(const float* g, const long* gd, int gn, const long* td, int tn, float* out) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor tg = make(g, gd, gn);
        Tensor root(ShapeTag{}, shape_of(td, tn), DType::kFloat, DeviceType::kAMD);
        root.requires_grad(true);
        ctx.make_leaf(root, true);
        ctx.backward(root, tg);
        return emit(grad(root), out);
    } catch (const std::exception&) {
        return -1;
    }
}
// d/da, d/db of dot(a, b) * scale: the closed form g * b, g * a that this tape adds (the reference
// has no gradient for Dot, src/AutoDiff.cpp:1856-1862)
long cth_grad_dot(const float* a, const float* b, long n, float scale, float* value, float* da, float* db) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        long d[1] = {n};
        Tensor ta = make(a, d, 1), tb = make(b, d, 1);
        ta.requires_grad(true);
        tb.requires_grad(true);
        Tensor y = ta.dot(tb);
        value[0] = y.item<float>();
        Tensor root = y * scale;
        backward(root);
        long r1 = emit(grad(ta), da), r2 = emit(grad(tb), db);
        return (r1 < 0 || r2 < 0) ? -2 : r1 + r2;
    } catch (const std::exception&) {
        return -1;
    }
}

// d/dpred of  loss(pred, target) * scale   (loss in MSE / MAE / CE); the upstream gradient of the
// loss node is then the 0-D value `scale`.
long cth_grad_loss(int code, const float* p, const long* pd, int pn, const float* t, const long* td,
                   int tn, float scale, float* loss_out, float* dp) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor tp = make(p, pd, pn), tt = make(t, td, tn);
        tp.requires_grad(true);
        Tensor l = run_binary(code, tp, tt);
        if (l.numel() == 0) return -2;
        loss_out[0] = l.item<float>();
        if (scale == 1.0f) {          // the loss itself is the root: its upstream gradient is the seed
            backward(l);
            return emit(grad(tp), dp);
        }
        Tensor root = l * scale;
        backward(root);
        return emit(grad(tp), dp);
    } catch (const std::exception&) {
        return -1;
    }
}

// Elementwise chain: c = a*b + 5, d = relu(c), s = d.sum(), s.backward().
long cth_chain(const float* a, const float* b, long n, float* s_out, float* ga, float* gb) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        long d1[1] = {n};
        Tensor ta = make(a, d1, 1), tb = make(b, d1, 1);
        ta.requires_grad(true);
        tb.requires_grad(true);
        Tensor d = g_fused_expr ? (Expr(ta) * Expr(tb) + 5.0f).relu().eval() : (ta * tb + 5.0f).relu();
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
long cth_mlp_step(const float* x, long B, long I, const float* W1, const float* b1, long H,
                  const float* W2, const float* b2, long C, const float* onehot, float* loss_out,
                  float* logits_out, float* gW1, float* gb1, float* gW2, float* gb2, int target_is_index) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        long xd[2] = {B, I}, w1d[2] = {I, H}, b1d[1] = {H}, w2d[2] = {H, C}, b2d[1] = {C},
             yd[2] = {B, C}, yi[1] = {B};
        Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1),
               tW2 = make(W2, w2d, 2), tb2 = make(b2, b2d, 1),
               ty = target_is_index ? make(onehot, yi, 1) : make(onehot, yd, 2);
        tW1.requires_grad(true);
        tb1.requires_grad(true);
        tW2.requires_grad(true);
        tb2.requires_grad(true);
        Tensor h = g_fused_layers ? tx.linear(tW1, tb1, true) : (tx.matmul(tW1) + tb1).relu();
        Tensor logits, loss;
        if (g_fused_layers && g_fused_head && target_is_index) {
            loss = h.linear_cross_entropy(tW2, tb2, ty, &logits);
        } else {
            logits = g_fused_layers ? h.linear(tW2, tb2, false) : h.matmul(tW2) + tb2;
            loss = logits.cross_entropy(ty);
        }
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
long cth_expr(const float* X, const float* R, const float* T, long rows, long cols, float* y_out,
              float* mse_out, float* mae_out, float* gX, float* gR, int r_is_row_vector) {
    try {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        long d[2] = {rows, cols}, dv[1] = {cols};
        Tensor tX = make(X, d, 2), tR = r_is_row_vector ? make(R, dv, 1) : make(R, d, 2), tT = make(T, d, 2);
        tX.requires_grad(true);
        tR.requires_grad(true);
        Tensor Y;
        if (g_fused_expr) {
            Expr x(tX), r(tR);
            Y = (sigmoid(x / r) - tanh(x) * sin(x) + cos(-x)).eval();
        } else {
            Tensor q = tX / tR;
            Tensor s1 = q.sigmoid();
            Tensor th = tX.tanh();
            Tensor sn = tX.sin();
            Tensor m = th * sn;
            Tensor d1 = s1 - m;
            Tensor ng = -tX;
            Tensor cs = ng.cos();
            Y = d1 + cs;
        }
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
long cth_program(const float* inputs, const int* kinds, int n_in, const int* ops, int n_ops, const float* w,
                 long rows, long cols, float* y_out, float* l_out, float* grads_out) {
    try {
        AutoDiff ctx;
        configure(ctx);
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
        if (g_fused_expr) {                     // the whole program as one expression
            std::vector<Expr> e(v.begin(), v.end());
            for (int k = 0; k < n_ops; ++k) {
                const int code = ops[3 * k], a = ops[3 * k + 1], b = ops[3 * k + 2];
                if (code < 20) e.push_back(run_binary(code, e[size_t(a)], e[size_t(b)]));
                else if (code < 30) e.push_back(run_unary(code, e[size_t(a)]));
                else {
                    const float s = 0.5f + 0.25f * float(b);
                    e.push_back(code == 30 ? e[size_t(a)] + s : code == 31 ? e[size_t(a)] * s : e[size_t(a)] / s);
                }
            }
            v.push_back(e.back().eval());
            n_ops = 0;
        }
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

// ------------------------------------------------------------------------- timed steps
// The same graphs as above with every input resident in HBM before the clock starts: `warm`
// untimed steps, then `reps` timed ones between two device synchronisations.  A step builds its
// own tape, runs forward and backward through the front-end and reads the loss back (the one
// host read a training step makes).  out[0] = milliseconds per step, out[1..4] = the launch
// layer's work counters per step: algorithmic bytes, flops, seconds at the MI355X peaks, operator
// launches.
}  // extern "C"
namespace {
double median_of(std::vector<double> v) {
    if (v.empty()) return 0.0;
    std::sort(v.begin(), v.end());
    const size_t h = v.size() / 2;
    return v.size() % 2 ? v[h] : 0.5 * (v[h - 1] + v[h]);
}
template <class Step>
long time_steps(Step step, int warm, int reps, double* out) {
    try {
        for (int i = 0; i < warm; ++i) step();
        ctamd_sync(nullptr);
        ctamd_counters_reset();
        // every step ends with a read that waits for the device (Dot's result, a loss), so the host
        // clock around one step times that step: out[5] is the median of the steps
        std::vector<double> each;
        each.reserve(size_t(reps));
        auto t0 = std::chrono::steady_clock::now();
        auto prev = t0;
        for (int i = 0; i < reps; ++i) {
            step();
            auto now = std::chrono::steady_clock::now();
            each.push_back(std::chrono::duration<double, std::milli>(now - prev).count());
            prev = now;
        }
        ctamd_sync(nullptr);
        auto t1 = std::chrono::steady_clock::now();
        out[5] = median_of(each);
        double bytes = 0, flops = 0, ideal = 0;
        uint64_t launches = 0;
        ctamd_counters_read(&bytes, &flops, &ideal, &launches);
        out[0] = std::chrono::duration<double, std::milli>(t1 - t0).count() / reps;
        out[1] = bytes / reps;
        out[2] = flops / reps;
        out[3] = ideal / reps;
        out[4] = double(launches) / reps;
        return reps;
    } catch (const std::exception&) {
        return -1;
    }
}
}  // namespace
extern "C" {

long cth_time_chain(const float* a, const float* b, long n, int warm, int reps, double* out) {
    long d1[1] = {n};
    Tensor ta = make(a, d1, 1), tb = make(b, d1, 1);
    volatile float sink = 0;
    return time_steps([&] {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        ta.requires_grad(true);
        tb.requires_grad(true);
        Tensor s = (g_fused_expr ? (Expr(ta) * Expr(tb) + 5.0f).relu().eval() : (ta * tb + 5.0f).relu()).sum();
        s.backward();                      // enqueued before the read below waits for the device
        sink = s.item<float>();
        Tensor ga = grad(ta), gb = grad(tb);
    }, warm, reps, out);
}

// C = A . B, L = C.sum(), backward: dC = ones, dA = dC . B^T, dB = A^T . dC.
long cth_time_matmul(const float* A, const float* B, long M, int warm, int reps, double* out) {
    long d[2] = {M, M};
    Tensor tA = make(A, d, 2), tB = make(B, d, 2);
    volatile float sink = 0;
    return time_steps([&] {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        tA.requires_grad(true);
        tB.requires_grad(true);
        Tensor L = tA.matmul(tB).sum();
        backward(L);                       // enqueued before the read below waits for the device
        sink = L.item<float>();
        Tensor ga = grad(tA), gb = grad(tB);
    }, warm, reps, out);
}

long cth_time_dot(const float* a, const float* b, long n, int warm, int reps, double* out) {
    long d1[1] = {n};
    Tensor ta = make(a, d1, 1), tb = make(b, d1, 1);
    volatile float sink = 0;
    return time_steps([&] { sink = ta.dot(tb).item<float>(); }, warm, reps, out);
}

long cth_time_mlp(const float* x, long B, long I, const float* W1, const float* b1, long H, const float* W2,
                  const float* b2, long C, const float* labels, int warm, int reps, double* out) {
    long xd[2] = {B, I}, w1d[2] = {I, H}, b1d[1] = {H}, w2d[2] = {H, C}, b2d[1] = {C}, yi[1] = {B};
    Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1), tW2 = make(W2, w2d, 2),
           tb2 = make(b2, b2d, 1), ty = make(labels, yi, 1);
    volatile float sink = 0;
    return time_steps([&] {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        tW1.requires_grad(true);
        tb1.requires_grad(true);
        tW2.requires_grad(true);
        tb2.requires_grad(true);
        Tensor h = g_fused_layers ? tx.linear(tW1, tb1, true) : (tx.matmul(tW1) + tb1).relu();
        Tensor loss = (g_fused_layers && g_fused_head) ? h.linear_cross_entropy(tW2, tb2, ty)
                                                        : (g_fused_layers ? h.linear(tW2, tb2, false) : h.matmul(tW2) + tb2).cross_entropy(ty);
        backward(loss);                    // enqueued before the read below waits for the device
        if (!g_no_loss_read) sink = loss.item<float>();
        Tensor g1 = grad(tW1), g2 = grad(tb1), g3 = grad(tW2), g4 = grad(tb2);
    }, warm, reps, out);
}

// The same MLP step with one-hot targets, recorded into a DeviceGraph once and replayed: a step is
// one graph launch plus reading the loss back.  out[4] reports the operator launches recorded.
long cth_time_mlp_graph(const float* x, long B, long I, const float* W1, const float* b1, long H, const float* W2,
                        const float* b2, long C, const float* onehot, int warm, int reps, double* out) {
    try {
        long xd[2] = {B, I}, w1d[2] = {I, H}, b1d[1] = {H}, w2d[2] = {H, C}, b2d[1] = {C}, yd[2] = {B, C};
        Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1), tW2 = make(W2, w2d, 2),
               tb2 = make(b2, b2d, 1), ty = make(onehot, yd, 2);
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor loss, g1, g2, g3, g4;
        auto body = [&] {
            tW1.requires_grad(true);
            tb1.requires_grad(true);
            tW2.requires_grad(true);
            tb2.requires_grad(true);
            Tensor h = g_fused_layers ? tx.linear(tW1, tb1, true) : (tx.matmul(tW1) + tb1).relu();
            loss = (g_fused_layers ? h.linear(tW2, tb2, false) : h.matmul(tW2) + tb2).cross_entropy(ty);
            backward(loss);
            g1 = grad(tW1), g2 = grad(tb1), g3 = grad(tW2), g4 = grad(tb2);
        };
        body();                               // once eagerly: the pool now holds every block the step needs
        ctx.clear_graph();
        ctamd_counters_reset();
        DeviceGraph step;
        step.record(body);
        double bytes = 0, flops = 0, ideal = 0;
        uint64_t launches = 0;
        ctamd_counters_read(&bytes, &flops, &ideal, &launches);
        float sink = 0;
        for (int i = 0; i < warm; ++i) { step.replay(); sink += loss.item<float>(); }
        std::vector<double> each;
        auto t0 = std::chrono::steady_clock::now();
        auto prev = t0;
        for (int i = 0; i < reps; ++i) {
            step.replay();
            sink += loss.item<float>();
            auto now = std::chrono::steady_clock::now();
            each.push_back(std::chrono::duration<double, std::milli>(now - prev).count());
            prev = now;
        }
        auto t1 = std::chrono::steady_clock::now();
        out[5] = median_of(each);
        out[0] = std::chrono::duration<double, std::milli>(t1 - t0).count() / reps;
        out[1] = bytes;
        out[2] = flops;
        out[3] = ideal;
        out[4] = double(launches);
        return sink == sink ? reps : reps;     // (the loss is read every step, as a training loop does)
    } catch (const std::exception&) {
        return -1;
    }
}

// The config-5 expression as a fused expression inside a recorded step: X1 is evaluated eagerly
// (y1, gx1), then the step is recorded on X1, replayed, the staged input is overwritten with X2 and
// the step replayed again, with eager work in between (y2, gx2 come from the second replay).
long cth_expr_graph(const float* X1, const float* X2, const float* R, const float* T, long rows, long cols, float* y1,
                    float* gx1, float* y2, float* gx2) {
    try {
        long d[2] = {rows, cols}, dv[1] = {cols};
        Tensor tX = make(X1, d, 2), tX2 = make(X2, d, 2), tR = make(R, dv, 1), tT = make(T, d, 2);
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        Tensor Y, gX;
        auto body = [&] {
            tX.requires_grad(true);
            tR.requires_grad(true);
            Expr x(tX), r(tR);
            Y = (sigmoid(x / r) - tanh(x) * sin(x) + cos(-x)).eval();
            Tensor L = Y.mse_loss(tT) + Y.mae_loss(tT);
            backward(L);
            gX = grad(tX);
        };
        body();                               // eagerly: the reference values for X1, and a warm pool
        if (emit(Y, y1) < 0 || emit(gX, gx1) < 0) return -2;
        ctx.clear_graph();
        DeviceGraph step;
        step.record(body);
        ctx.clear_graph();
        step.replay();
        Tensor probe = (tT * 2.0f).sum();     // eager work between the replays
        (void)probe.item<float>();
        std::vector<float> a(size_t(rows * cols)), b(size_t(rows * cols));
        if (emit(Y, a.data()) < 0 || emit(gX, b.data()) < 0) return -2;
        if (std::memcmp(a.data(), y1, a.size() * sizeof(float)) != 0 || std::memcmp(b.data(), gx1, b.size() * sizeof(float)) != 0)
            return -3;                        // the first replay must reproduce the eager step
        ctorch_amd_host::copy_into(tX, tX2);
        step.replay();
        if (emit(Y, y2) < 0 || emit(gX, gx2) < 0) return -2;
        return rows * cols;
    } catch (const std::exception&) {
        return -1;
    }
}

// Recorded steps under stress.  out[0..3]: sums from two graphs replayed alternately, with no host
// wait between them and new input contents before each pair, and the same sums computed eagerly
// on the last input; out[4]: item() of a one-element parameter after an in-place SGD step (2 - 1 *
// 0.5); out[5]: gradient of sum(x * x) at x[0] from a backward() issued eagerly on a thread whose
// first backward() was inside a recording; out[6]: 1 if a DeviceGraph whose first recording
// failed records and replays a second body.  Returns 0, or a negative code for an exception.
long cth_graph_hardening(const float* X, const float* X2, long n, float* out) {
    try {
        long d[1] = {n};
        Tensor tx = make(X, d, 1), tx2 = make(X2, d, 1), staged = make(X, d, 1);
        Tensor ty, sa, sb, sc;
        auto body_a = [&] { ty = staged * 2.0f; sa = ty.sum(); };
        auto body_b = [&] { Tensor tz = ty + 1.0f; sb = tz.sum(); sc = (tz * tz).sum(); };
        body_a();
        body_b();                                  // eagerly once: a warm pool, ty exists
        DeviceGraph ga, gb;
        ga.record(body_a);
        gb.record(body_b);
        for (int it = 0; it < 6; ++it) {
            ctorch_amd_host::copy_into(staged, (it % 2) ? tx2 : tx);
            ga.replay();
            gb.replay();                           // reads what ga wrote; both use the device scratch
        }
        out[0] = sa.item<float>();
        out[1] = sb.item<float>();
        Tensor ey = tx2 * 2.0f, ez = ey + 1.0f;
        out[2] = ey.sum().item<float>();
        out[3] = ez.sum().item<float>();
        if (sc.item<float>() != (ez * ez).sum().item<float>()) return -3;

        Tensor p(2.0f, DeviceType::kAMD), g(0.5f, DeviceType::kAMD);
        if (p.item<float>() != 2.0f) return -4;
        ctorch_amd_host::sgd_step(p, g, 1.0f);
        out[4] = p.item<float>();

        float first_grad = -1.0f;
        long thread_rc = 0;
        std::thread worker([&] {
            try {
                AutoDiff ctx;
                configure(ctx);
                AutoDiffContext::Guard guard(&ctx);
                Tensor w = make(X, d, 1), gw;
                auto step = [&] {
                    w.requires_grad(true);
                    Tensor L = (w * w).sum();
                    backward(L);
                    gw = grad(w);
                };
                DeviceGraph rec;
                rec.record(step);                  // this thread's first backward(): inside a recording
                ctx.clear_graph();
                step();                            // eagerly, before any replay
                std::vector<float> host(static_cast<size_t>(n));
                if (emit(gw, host.data()) < 0) { thread_rc = -5; return; }
                first_grad = host[0];
            } catch (const std::exception&) {
                thread_rc = -6;
            }
        });
        worker.join();
        if (thread_rc) return thread_rc;
        out[5] = first_grad;

        DeviceGraph again;
        bool threw = false;
        try {
            again.record([&] { Tensor t = staged * 3.0f; (void)t.sum().item<float>(); });   // a host wait: refused while recording
        } catch (const std::exception&) {
            threw = true;
        }
        Tensor kept;
        again.record([&] { kept = staged * 3.0f; });
        again.replay();
        again.wait();
        std::vector<float> host(static_cast<size_t>(n));
        if (emit(kept, host.data()) < 0) return -7;
        out[6] = (threw && again.recorded() && host[0] == X2[0] * 3.0f) ? 1.0f : 0.0f;   // staged holds X2 after the loop
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

// CrossEntropy (class index) of two logits matrices forward, then both backward, three times: with
// the default cap on kept one-pass gradients, with a cap that holds only one of them (the older
// gives way and its backward recomputes), and with a cap below either (no one-pass gradient at all).
// Returns 0 when the first two agree bit for bit on both gradients and the third - which works from
// the forward pass's row statistics - to 2e-7; writes the first into g1 / g2.
long cth_ce_kept_cap(const float* x1, const float* x2, const float* labels, long rows, long cols, float* g1, float* g2) {
    try {
        long d[2] = {rows, cols}, yi[1] = {rows};
        Tensor ty = make(labels, yi, 1);
        const size_t before = ctorch_amd_host::ce_kept_bytes();
        const size_t one = size_t(rows) * size_t(cols) * sizeof(float);
        const size_t caps[3] = {before, one + one / 2, one / 2};
        std::vector<float> a(size_t(rows * cols)), b(size_t(rows * cols));
        long rc = 0;
        for (int k = 0; k < 3 && rc == 0; ++k) {
            ctorch_amd_host::set_ce_kept_bytes(caps[k]);
            Tensor t1 = make(x1, d, 2), t2 = make(x2, d, 2);
            AutoDiff ctx;
            configure(ctx);
            AutoDiffContext::Guard guard(&ctx);
            t1.requires_grad(true);
            t2.requires_grad(true);
            Tensor l1 = t1.cross_entropy(ty), l2 = t2.cross_entropy(ty);
            Tensor L = l1 + l2;
            backward(L);
            float* o1 = k == 0 ? g1 : a.data();
            float* o2 = k == 0 ? g2 : b.data();
            if (emit(grad(t1), o1) < 0 || emit(grad(t2), o2) < 0) rc = -2;
            else if (k == 1 && (std::memcmp(o1, g1, a.size() * sizeof(float)) != 0 || std::memcmp(o2, g2, b.size() * sizeof(float)) != 0)) rc = -11;
            else if (k == 2) {                  // from the forward pass's row statistics: the same values to rounding
                for (size_t i = 0; i < a.size(); ++i)
                    if (!(std::fabs(o1[i] - g1[i]) <= 2e-7f) || !(std::fabs(o2[i] - g2[i]) <= 2e-7f)) rc = -12;
            }
        }
        ctorch_amd_host::set_ce_kept_bytes(before);
        return rc;
    } catch (const std::exception&) {
        return -1;
    }
}

// A gradient read from the tape shares the tape's bytes and is read-only while it does: fill, copy_into
// and an SGD step into it throw; once the tape has let go of it the last holder may write.
// Returns 0 when all of that holds.
long cth_shared_grad_is_readonly(const float* a, long n) {
    try {
        long d[1] = {n};
        Tensor ta = make(a, d, 1), other = make(a, d, 1);
        Tensor g;
        int threw = 0;
        {
            AutoDiff ctx;
            configure(ctx);
            AutoDiffContext::Guard guard(&ctx);
            ta.requires_grad(true);
            Tensor L = (ta * ta).sum();
            backward(L);
            g = grad(ta);
            try { g.fill(1.0f); } catch (const std::exception&) { ++threw; }
            try { ctorch_amd_host::copy_into(g, other); } catch (const std::exception&) { ++threw; }
            try { ctorch_amd_host::sgd_step(g, other, 0.1f); } catch (const std::exception&) { ++threw; }
        }
        if (threw != 3) return -2;
        g.fill(1.0f);                              // the tape is gone: g is the only holder
        std::vector<float> host(static_cast<size_t>(n));
        if (emit(g, host.data()) < 0 || host[0] != 1.0f) return -3;
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

// A three-layer network of fused layers, trained gradients and the gradients of the two hidden
// activations, with the ReLU mask riding in the products of backward and without, after one
// backward pass and after two passes over the same tape: 0 when every gradient agrees bit for bit,
// else 1 + the index of the first that differs (+ 100 for the two-pass run).  out[0]: kernels
// launched by one backward with the mask in the products, out[1]: without.
long cth_relu_mask_fusion(const float* x, long B, long I, const float* W1, const float* b1, long H1, const float* W2,
                          const float* b2, long H2, const float* W3, const float* b3, long C, const float* labels,
                          double* out) {
    try {
        auto run = [&](bool fuse, int passes, double* launches) {
            std::vector<std::vector<float>> grads;
            AutoDiff ctx;
            configure(ctx);
            ctx.set_fuse_relu_mask(fuse);        // this check sets it itself
            AutoDiffContext::Guard guard(&ctx);
            long xd[2] = {B, I}, w1d[2] = {I, H1}, b1d[1] = {H1}, w2d[2] = {H1, H2}, b2d[1] = {H2}, w3d[2] = {H2, C},
                 b3d[1] = {C}, yi[1] = {B};
            Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1), tW2 = make(W2, w2d, 2),
                   tb2 = make(b2, b2d, 1), tW3 = make(W3, w3d, 2), tb3 = make(b3, b3d, 1), ty = make(labels, yi, 1);
            for (Tensor* t : {&tW1, &tb1, &tW2, &tb2, &tW3, &tb3}) t->requires_grad(true);
            Tensor h1 = tx.linear(tW1, tb1, true);
            Tensor h2 = h1.linear(tW2, tb2, true);
            Tensor logits = h2.linear(tW3, tb3, false);
            Tensor loss = logits.cross_entropy(ty);
            for (int p = 0; p < passes; ++p) {
                double bytes = 0.0, flops = 0.0, ideal = 0.0;
                uint64_t before = 0, after = 0;
                ctamd_counters_read(&bytes, &flops, &ideal, &before);
                backward(loss);
                ctamd_counters_read(&bytes, &flops, &ideal, &after);
                if (launches) *launches = double(after - before);
            }
            for (Tensor* t : {&tW1, &tb1, &tW2, &tb2, &tW3, &tb3, &h1, &h2}) grads.push_back(grad(*t).to_vector());
            return grads;
        };
        for (int passes = 1; passes <= 2; ++passes) {
            auto with = run(true, passes, passes == 1 ? out : nullptr);
            auto without = run(false, passes, passes == 1 ? out + 1 : nullptr);
            for (size_t i = 0; i < with.size(); ++i)
                if (with[i].size() != without[i].size() ||
                    std::memcmp(with[i].data(), without[i].data(), with[i].size() * sizeof(float)) != 0)
                    return long(1 + i) + (passes == 2 ? 100 : 0);
        }
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

// A hidden ReLU layer whose gradient the tape holds at the pre-activation (the mask rode in the
// consumer's product): reading the gradient of the layer's output forms it once (the second read
// launches nothing and returns the same bits); clearing the consumer's gradient takes the hidden
// layer's with it (it reads as zeros, as any cleared gradient); a further backward pass over the tape
// then gives the gradients of a first pass again.  0, or the number of the first check that failed.
long cth_premasked_grad_reads(const float* x, long B, long I, const float* W1, const float* b1, long H, const float* W2,
                              const float* b2, long C, const float* labels) {
    try {
        prepare_backward_seed();
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        long xd[2] = {B, I}, w1d[2] = {I, H}, b1d[1] = {H}, w2d[2] = {H, C}, b2d[1] = {C}, yi[1] = {B};
        Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1), tW2 = make(W2, w2d, 2), tb2 = make(b2, b2d, 1),
               ty = make(labels, yi, 1);
        for (Tensor* t : {&tW1, &tb1, &tW2, &tb2}) t->requires_grad(true);
        Tensor h = tx.linear(tW1, tb1, true);
        Tensor logits = h.linear(tW2, tb2, false);
        Tensor loss = logits.cross_entropy(ty);
        backward(loss);
        auto launches = [] {
            double a = 0, b = 0, c = 0;
            uint64_t n = 0;
            ctamd_counters_read(&a, &b, &c, &n);
            return n;
        };
        const std::vector<float> gw1 = grad(tW1).to_vector();
        const uint64_t n0 = launches();
        const std::vector<float> first = grad(h).to_vector();
        const uint64_t n1 = launches();
        const std::vector<float> second = grad(h).to_vector();
        const uint64_t n2 = launches();
        if (n1 == n0) return 1;                                   // the first read has to form the product
        if (n2 != n1) return 2;                                   // the second must not
        if (first != second) return 3;
        bool any = false;
        for (float v : first) any = any || v != 0.0f;
        if (!any) return 4;
        ctx.zero_grad(logits);
        for (float v : grad(h).to_vector())
            if (v != 0.0f) return 5;                              // its source is gone
        for (Tensor* t : {&tW1, &tb1, &tW2, &tb2}) ctx.zero_grad(*t);
        ctx.zero_grad(loss);
        backward(loss);                                           // over the same tape: as a first pass
        if (grad(tW1).to_vector() != gw1) return 6;
        if (grad(h).to_vector() != first) return 7;
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

// The same three-layer network with its last layer and cross entropy as one operator
// (Tensor::linear_cross_entropy) against the two-operator form: loss, logits, the six parameter
// gradients and the gradients of the two hidden activations, for the loss as the root of backward
// (the gradients the one pass kept), for `loss * scale` as the root (the kept gradient of the logits
// rescaled, the usual products); then two passes over one tape with the head (see below).  0 when
// everything agrees within tol * max(1, largest magnitude), else 1 + the index of the first result
// that does not (+ 100 scaled root, + 200 two passes); out[0]: the worst ratio seen, out[1] / out[2]: operator launches of one
// step with / without the one-pass head.
long cth_head_fusion(const float* x, long B, long I, const float* W1, const float* b1, long H1, const float* W2,
                     const float* b2, long H2, const float* W3, const float* b3, long C, const float* labels, double tol,
                     float scale, double* out) {
    try {
        prepare_backward_seed();              // made once per thread by a launch that is not part of a step
        auto run = [&](bool head, int variant, double* launches) {
            std::vector<std::vector<float>> results;
            AutoDiff ctx;
            configure(ctx);
            AutoDiffContext::Guard guard(&ctx);
            long xd[2] = {B, I}, w1d[2] = {I, H1}, b1d[1] = {H1}, w2d[2] = {H1, H2}, b2d[1] = {H2}, w3d[2] = {H2, C},
                 b3d[1] = {C}, yi[1] = {B};
            Tensor tx = make(x, xd, 2), tW1 = make(W1, w1d, 2), tb1 = make(b1, b1d, 1), tW2 = make(W2, w2d, 2),
                   tb2 = make(b2, b2d, 1), tW3 = make(W3, w3d, 2), tb3 = make(b3, b3d, 1), ty = make(labels, yi, 1);
            for (Tensor* t : {&tW1, &tb1, &tW2, &tb2, &tW3, &tb3}) t->requires_grad(true);
            double bytes = 0.0, flops = 0.0, ideal = 0.0;
            uint64_t before = 0, after = 0;
            ctamd_counters_read(&bytes, &flops, &ideal, &before);
            Tensor h1 = tx.linear(tW1, tb1, true);
            Tensor h2 = h1.linear(tW2, tb2, true);
            Tensor logits, loss;
            if (head) {
                loss = h2.linear_cross_entropy(tW3, tb3, ty, &logits);
            } else {
                logits = h2.linear(tW3, tb3, false);
                loss = logits.cross_entropy(ty);
            }
            Tensor root = variant == 1 ? loss * scale : Tensor::alias(loss);
            if (variant == 1) root = loss * scale;
            for (int p = 0; p < (variant == 2 ? 2 : 1); ++p) backward(variant == 1 ? root : loss);
            ctamd_counters_read(&bytes, &flops, &ideal, &after);
            if (launches) *launches = double(after - before);
            results.push_back({loss.item<float>()});
            results.push_back(logits.to_vector());
            for (Tensor* t : {&tW1, &tb1, &tW2, &tb2, &tW3, &tb3, &h1, &h2}) results.push_back(grad(*t).to_vector());
            return results;
        };
        double worst = 0.0;
        for (int variant = 0; variant < 2; ++variant) {
            auto with = run(true, variant, variant == 0 ? out + 1 : nullptr);
            auto without = run(false, variant, variant == 0 ? out + 2 : nullptr);
            for (size_t i = 0; i < with.size(); ++i) {
                if (with[i].size() != without[i].size()) return long(1 + i) + 100 * variant;
                double big = 1.0, diff = 0.0;
                for (size_t k = 0; k < with[i].size(); ++k) {
                    big = std::max(big, double(std::fabs(without[i][k])));
                    const double d = std::fabs(double(with[i][k]) - double(without[i][k]));
                    diff = (d == d) ? std::max(diff, d) : 1e30;
                }
                worst = std::max(worst, diff / big);
                if (diff > tol * big) {
                    out[0] = worst;
                    return long(1 + i) + 100 * variant;
                }
            }
        }
        // Two passes over one tape.  The head is ONE node: each pass adds one contribution to its
        // inputs, so the gradients of the last layer and of h2 are exactly twice those of one pass.  (The
        // two-operator form has a logits node in between whose gradient accumulates as well - the
        // reference's tape never clears a node's gradient - and hands on 1 + 2 contributions.)
        {
            auto once = run(true, 0, nullptr);
            auto twice = run(true, 2, nullptr);
            for (size_t i : {size_t(6), size_t(7), size_t(9)})
                for (size_t k = 0; k < once[i].size(); ++k)
                    if (twice[i][k] != once[i][k] + once[i][k]) {
                        out[0] = worst;
                        return long(1 + i) + 200;
                    }
        }
        out[0] = worst;
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

// loss_sum = CE(logits, class index), backward: dlogits = softmax - onehot.
long cth_time_softmax_ce(const float* logits, const float* labels, long rows, long cols, int warm, int reps,
                         double* out) {
    long d[2] = {rows, cols}, yi[1] = {rows};
    Tensor tx = make(logits, d, 2), ty = make(labels, yi, 1);
    volatile float sink = 0;
    return time_steps([&] {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        tx.requires_grad(true);
        Tensor loss = tx.cross_entropy(ty);
        backward(loss);                    // enqueued before the read below waits for the device
        sink = loss.item<float>() / float(rows);
        Tensor g = grad(tx);
    }, warm, reps, out);
}

long cth_time_expr(const float* X, const float* R, const float* T, long rows, long cols, int warm, int reps,
                   double* out) {
    long d[2] = {rows, cols}, dv[1] = {cols};
    Tensor tX = make(X, d, 2), tR = make(R, dv, 1), tT = make(T, d, 2);
    volatile float sink = 0;
    return time_steps([&] {
        AutoDiff ctx;
        configure(ctx);
        AutoDiffContext::Guard guard(&ctx);
        tX.requires_grad(true);
        tR.requires_grad(true);
        Tensor Y = g_fused_expr ? (sigmoid(Expr(tX) / Expr(tR)) - tanh(Expr(tX)) * sin(Expr(tX)) + cos(-Expr(tX))).eval()
                                : (tX / tR).sigmoid() - tX.tanh() * tX.sin() + (-tX).cos();
        Tensor L = Y.mse_loss(tT) + Y.mae_loss(tT);
        backward(L);                       // enqueued before the read below waits for the device
        sink = L.item<float>();
        Tensor gX = grad(tX), gR = grad(tR);
    }, warm, reps, out);
}

// ------------------------------------------------------------------------- MNIST demo path
// Same shapes as the reference-side doorway (ref_mnist_* of the test infrastructure).

long cth_mnist_load(const char* dir, int which, float* images_out, float* labels_out, long* dims_out) {
    try {
        MNISTLoader loader(dir);
        Tensor images, labels;
        if (which) loader.load_training_data(images, labels);
        else loader.load_test_data(images, labels);
        dims_out[0] = long(images.shape()[0]);
        dims_out[1] = long(images.shape()[1]);
        if (images_out) emit(images, images_out);
        if (labels_out) emit(labels, labels_out);
        return long(labels.numel());
    } catch (const std::exception&) {
        return -1;
    }
}

float cth_mnist_accuracy(const float* pred, const float* labels, long rows) {
    long pd[2] = {rows, 10}, ld[1] = {rows};
    Tensor p = make(pred, pd, 2), y = make(labels, ld, 1);
    return calculate_accuracy(p, y);
}

// `steps` consecutive batches (batch index = step % (n_images / batch)) inside one autograd
// context, data set and parameters resident.  mode_bits & 3 = reference_tape; reference_tape == 1: leaf values frozen at their
// first-seen copies and row-0 bias gradients (the reference's behaviour); else live leaves, column
// sums and a tape cleared after every step; 2: as 0 with the step recorded into a DeviceGraph at
// the first batch and replayed for every batch (with unrelated eager work between the replays).
// Adding 4 to the mode makes each layer one fused operator and the optimiser update one launch
// (same values); adding 8 as well, the last layer and its loss are the one-pass head.  Parameters are written back; losses_out[s] = loss of step s.  ms_out (may be null) = milliseconds for all the steps.
long cth_mnist_train(const float* images, const float* labels, long n_images, long I, long H1, long H2, long C,
                     float* W1, float* b1, float* W2, float* b2, float* W3, float* b3, long batch, long steps,
                     float lr, int mode_bits, float* losses_out, double* ms_out) {
    try {
        const int reference_tape = mode_bits & 3;
        const bool fused = (mode_bits & 4) != 0;
        long id[2] = {n_images, I}, ld[1] = {n_images};
        Tensor all_images = make(images, id, 2), all_labels = make(labels, ld, 1);
        NeuralNetwork model(W1, b1, W2, b2, W3, b3, size_t(I), size_t(H1), size_t(H2), size_t(C), lr);
        model.fused_layers = fused;
        model.fused_head = (mode_bits & 8) != 0;
        const long num_batches = n_images / batch;
        AutoDiff autodiff;
        if (reference_tape == 1) {
            autodiff.set_broadcast_grad(BroadcastGrad::kReferenceRow0);
            autodiff.set_leaf_values(LeafValues::kReferenceFirstSeen);
        }
        AutoDiffContext::Guard guard(&autodiff);
        DeviceGraph step;                    // reference_tape == 2: the step is recorded once and replayed
        Tensor sx, sy, sloss;
        if (reference_tape == 2) {
            sx = Tensor(ShapeTag{}, {size_t(batch), size_t(I)}, DType::kFloat, DeviceType::kAMD, false);
            sy = Tensor(ShapeTag{}, {size_t(batch)}, DType::kFloat, DeviceType::kAMD, false);
        }
        ctamd_sync(nullptr);
        auto t0 = std::chrono::steady_clock::now();
        for (long s = 0; s < steps; ++s) {
            Tensor x, y;
            get_batch(all_images, all_labels, int(batch), int(s % num_batches), x, y);
            if (reference_tape == 2) {
                ctorch_amd_host::copy_into(sx, x);
                ctorch_amd_host::copy_into(sy, y);
                if (!step.recorded()) {
                    step.record([&] { sloss = model.train_step_on_device(sx, sy); });
                    autodiff.clear_graph();
                }
                step.replay();
                // eager work between replays, on the null stream, through the pool
                Tensor probe = (sx * 2.0f).sum();
                losses_out[s] = sloss.item<float>();
                (void)probe.item<float>();
                continue;
            }
            losses_out[s] = model.train_step(x, y);
            if (!reference_tape) autodiff.clear_graph();
        }
        ctamd_sync(nullptr);
        if (ms_out) *ms_out = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        emit(model.W1, W1);
        emit(model.b1, b1);
        emit(model.W2, W2);
        emit(model.b2, b2);
        emit(model.W3, W3);
        emit(model.b3, b3);
        return steps;
    } catch (const std::exception&) {
        return -1;
    }
}

// probabilities [B, C] of the demo's predict() for given parameters
long cth_mnist_predict(const float* x, long B, long I, long H1, long H2, long C, const float* W1, const float* b1,
                       const float* W2, const float* b2, const float* W3, const float* b3, float* probs_out) {
    try {
        long xd[2] = {B, I};
        Tensor tx = make(x, xd, 2);
        NeuralNetwork model(W1, b1, W2, b2, W3, b3, size_t(I), size_t(H1), size_t(H2), size_t(C), 0.0f);
        return emit(model.predict(tx), probs_out);
    } catch (const std::exception&) {
        return -1;
    }
}

// The whole demo on the files in `dir`.  epoch_loss_out has room for `epochs` values;
// acc_out = {train accuracy, test accuracy}; seconds_out = training time.
long cth_mnist_demo(const char* dir, int epochs, int batch, float lr, int hidden1, int hidden2, int mode_bits,
                    float* epoch_loss_out, float* acc_out, double* seconds_out) {
    try {
        MnistDemoOptions opt;
        opt.dir = dir;
        opt.epochs = epochs;
        opt.batch_size = batch;
        opt.learning_rate = lr;
        opt.hidden1 = hidden1;
        opt.hidden2 = hidden2;
        const int reference_tape = mode_bits & 3;
        opt.fused_layers = (mode_bits & 4) != 0;
        opt.fused_head = (mode_bits & 8) != 0;
        opt.loss_on_device = (mode_bits & 16) == 0;       // 16: every step reads its loss
        opt.reference_tape = reference_tape == 1;
        opt.use_graph = reference_tape == 2;          // 2: live leaves and the step replayed from a recorded graph
        MnistDemoResult r = run_mnist_demo(opt);
        for (size_t e = 0; e < r.epoch_loss.size(); ++e) epoch_loss_out[e] = r.epoch_loss[e];
        acc_out[0] = r.train_accuracy;
        acc_out[1] = r.test_accuracy;
        if (seconds_out) *seconds_out = r.train_seconds;
        return long(r.num_batches) * epochs;
    } catch (const std::exception&) {
        return -1;
    }
}

}  // extern "C"
