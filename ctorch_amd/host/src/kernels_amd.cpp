// The AMD column of the scheduler: <Op>_AMD_kernel shims with the reference's kernel signatures
// (src/kernels/kernels.h:23,31).  Each one checks what its CPU-BASIC twin checks, allocates the
// result in HBM and calls the extern "C" launch layer on the default stream.  Launches are
// asynchronous; the host only waits where it reads a value (item(), to(kCPU), the CrossEntropy
// label-range flag).
#include "kernels.h"

#include "AutoDiff.h"

#include "ctorch_amd.h"

namespace ctorch_amd_host {
namespace {

constexpr ErrorPlatform kP = ErrorPlatform::kAMD;

void run(int rc, const char* what) {
    if (rc == CTAMD_OK) return;
    ErrorType t = rc == CTAMD_EINVAL ? ErrorType::DIMENSION : rc == CTAMD_ENOMEM ? ErrorType::MEMORY : ErrorType::KERNEL_LAUNCH;
    Ctorch_Error::throwException(kP, t, std::string(what) + ": " + ctamd_last_error());
}

void check_device(const Tensor& a, const char* who) {
    if (a.device() != DeviceType::kAMD)
        Ctorch_Error::throwException(DeviceTypeToErrorPlatform(a.device()), ErrorType::DEVICE_COMPAT,
                                     std::string(who) + ": tensor is not on the AMD device");
    if (a.dtype() != DType::kFloat)
        Ctorch_Error::throwException(kP, ErrorType::DATATYPE, std::string(who) + ": only float32 tensors");
}

Tensor like(const Tensor& a) { return Tensor(ShapeTag{}, a.sizes(), DType::kFloat, DeviceType::kAMD, false); }
Tensor scalar0d() { return Tensor(ShapeTag{}, {}, DType::kFloat, DeviceType::kAMD, false); }

typedef int (*Bin)(const float*, const float*, float*, size_t, void*);
typedef int (*BinRow)(const float*, const float*, float*, size_t, size_t, void*);
typedef int (*Un)(const float*, float*, size_t, void*);

struct BinaryFamily {
    const char* name;
    Bin same, bscalar;
    BinRow rowbcast;
};
const BinaryFamily kAdd{"Add_AMD_kernel", ctamd_add_f32, ctamd_add_bscalar_f32, ctamd_add_rowbcast_f32};
const BinaryFamily kSub{"Sub_AMD_kernel", ctamd_sub_f32, ctamd_sub_bscalar_f32, ctamd_sub_rowbcast_f32};
const BinaryFamily kMul{"Mul_AMD_kernel", ctamd_mul_f32, ctamd_mul_bscalar_f32, ctamd_mul_rowbcast_f32};
const BinaryFamily kDiv{"Div_AMD_kernel", ctamd_div_f32, ctamd_div_bscalar_f32, ctamd_div_rowbcast_f32};

bool row_broadcastable(const Tensor& a, const Tensor& b) {
    return b.sizes().size() == 1 && a.sizes().size() == 2 && b.sizes()[0] == a.sizes()[1];
}

// Shape rules: same shape; b with one element (Add_BASIC_kernel.cpp:23,48-53; 0-D operands of
// Sub / Mul: Sub_BASIC_kernel.cpp:25-32); a [rows, cols] with b [cols] (Add_BASIC_kernel.cpp:27-29).
// A 0-D `a` against a larger `b` follows the reference per op: Sub and Mul broadcast it, Add and
// Div do not support it.
Tensor elementwise(const BinaryFamily& f, const Tensor& a, const Tensor& b, bool a_scalar_ok) {
    check_device(a, f.name);
    check_device(b, f.name);
    if (a.sizes() == b.sizes()) {
        Tensor r = like(a);
        run(f.same(a.fptr(), b.fptr(), r.fptr(), a.numel(), current_stream()), f.name);
        return r;
    }
    if (b.numel() == 1) {
        Tensor r = like(a);
        run(f.bscalar(a.fptr(), b.fptr(), r.fptr(), a.numel(), current_stream()), f.name);
        return r;
    }
    if (row_broadcastable(a, b)) {
        Tensor r = like(a);
        run(f.rowbcast(a.fptr(), b.fptr(), r.fptr(), a.sizes()[0], a.sizes()[1], current_stream()), f.name);
        return r;
    }
    if (a_scalar_ok && a.dim() == 0) {
        Tensor r = like(b);
        if (&f == &kMul) run(ctamd_mul_bscalar_f32(b.fptr(), a.fptr(), r.fptr(), b.numel(), current_stream()), f.name);
        else run(ctamd_rsub_ascalar_f32(a.fptr(), b.fptr(), r.fptr(), b.numel(), current_stream()), f.name);
        return r;
    }
    Ctorch_Error::throwException(kP, ErrorType::DIMENSION, std::string(f.name) + ": shapes differ and cannot be broadcast");
}

Tensor map(Un fn, const char* name, const Tensor& a) {
    check_device(a, name);
    Tensor r = like(a);
    run(fn(a.fptr(), r.fptr(), a.numel(), current_stream()), name);
    return r;
}

Tensor reduce2(int (*fn)(const float*, const float*, float*, size_t, void*), const char* name, const Tensor& a,
               const Tensor& b, bool same_shape) {
    check_device(a, name);
    check_device(b, name);
    if (same_shape ? a.sizes() != b.sizes() : a.numel() != b.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, std::string(name) + ": operand sizes differ");
    Tensor r = scalar0d();
    run(fn(a.fptr(), b.fptr(), r.fptr(), a.numel(), current_stream()), name);
    return r;
}

void rows_cols(const Tensor& a, size_t& rows, size_t& cols) {
    if (a.dim() == 1) { rows = 1; cols = a.sizes()[0]; }
    else { rows = a.sizes()[0]; cols = a.sizes()[1]; }
}

// a contiguous device tensor of any dtype
void check_on_device(const Tensor& a, const char* who) {
    if (a.device() != DeviceType::kAMD)
        Ctorch_Error::throwException(DeviceTypeToErrorPlatform(a.device()), ErrorType::DEVICE_COMPAT,
                                     std::string(who) + ": tensor is not on the AMD device");
    if (!a.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::TENSOR_STATE, std::string(who) + ": a contiguous tensor is needed");
}

bool g_ce_one_pass = true;

}  // namespace

// ------------------------------------------------------------------ helpers for Tensor / tape
void set_ce_one_pass(bool on) { g_ce_one_pass = on; }
namespace {
struct DeferredCheck {
    Tensor status;          // four bytes on the device: nonzero = the condition was met
    std::string message;
};
thread_local std::vector<DeferredCheck> t_deferred;
}  // namespace
void defer_status_check(const Tensor& status, const std::string& message) { t_deferred.push_back({Tensor::alias(status), message}); }
void drop_deferred_checks() { t_deferred.clear(); }
void run_deferred_checks() {
    std::vector<DeferredCheck> pending;
    pending.swap(t_deferred);
    for (const DeferredCheck& c : pending) {
        int32_t v = 0;
        device_copy_d2h(&v, c.status.fptr(), sizeof(v));
        if (v) Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, c.message);
    }
}
bool g_ce_deferred_check = false;
void set_ce_deferred_label_check(bool on) { g_ce_deferred_check = on; }
bool ce_deferred_label_check() { return g_ce_deferred_check; }
// Kept one-pass CrossEntropy gradients are as large as their logits and wait for a backward() that
// may never come (a forward pass under a tape that is then dropped): together they hold at most
// this many bytes, the oldest give way first, and logits larger than the cap get no such gradient.
size_t g_ce_kept_cap = size_t(4) << 30;
void set_ce_kept_bytes(size_t cap) { g_ce_kept_cap = cap; }
size_t ce_kept_bytes() { return g_ce_kept_cap; }
bool ce_one_pass() { return g_ce_one_pass; }

void fill_typed(void* device_ptr, DType dtype, double v, size_t n) {
    run(ctamd_fill_typed(device_ptr, int(dtype), v, n, current_stream()), "zero / ones");
}
Tensor cast_from_float(const Tensor& a, DType to) {
    check_device(a, "to(dtype)");                                       // src/Tensor.cpp:206: conversions start from float only
    if (!a.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::TENSOR_STATE, "to(dtype): a contiguous tensor is needed");
    Tensor r(ShapeTag{}, a.sizes(), to, DeviceType::kAMD, false);
    run(ctamd_cast_from_f32(a.fptr(), r.raw_ptr(), int(to), a.numel(), current_stream()), "to(dtype)");
    return r;
}
Tensor scalar_op(const Tensor& a, float s, op which) {
    if (a.dtype() != DType::kFloat) {
        // the typed arms of src/Tensor.cpp:766-786, :870-890, :933-953; anything else is refused as there
        if ((a.dtype() != DType::kDouble && a.dtype() != DType::kInt && a.dtype() != DType::kLong) || which == op::Sub)
            Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "tensor (op) float: unsupported dtype");
        check_on_device(a, "tensor (op) float");
        Tensor r(ShapeTag{}, a.sizes(), a.dtype(), DeviceType::kAMD, false);
        const int code = which == op::Add ? CTAMD_TS_ADD : which == op::Mul ? CTAMD_TS_MUL : CTAMD_TS_DIV;
        run(ctamd_scalar_op_typed(a.raw_ptr(), r.raw_ptr(), int(a.dtype()), code, s, a.numel(), current_stream()), "tensor (op) float");
        return r;
    }
    check_device(a, "tensor (op) float");
    Tensor r = like(a);
    int rc = which == op::Add ? ctamd_add_scalar_f32(a.fptr(), s, r.fptr(), a.numel(), current_stream())
           : which == op::Sub ? ctamd_sub_scalar_f32(a.fptr(), s, r.fptr(), a.numel(), current_stream())
           : which == op::Mul ? ctamd_mul_scalar_f32(a.fptr(), s, r.fptr(), a.numel(), current_stream())
                              : ctamd_div_scalar_f32(a.fptr(), s, r.fptr(), a.numel(), current_stream());
    run(rc, "tensor (op) float");
    return r;
}
Tensor compare_op(int cmp, const Tensor& a, const Tensor* b, float s) {
    check_device(a, "comparison");
    if (a.dtype() != DType::kFloat || !a.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::DATATYPE, "comparison: a contiguous float tensor is needed");
    if (b) {
        check_device(*b, "comparison");
        if (a.sizes() != b->sizes())                                    // src/Tensor.cpp:1124-1126
            Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DIMENSION, "comparison: tensor shapes differ");
        if (a.dtype() != b->dtype() || !b->is_contiguous())             // :1129-1131
            Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "comparison: tensor dtypes differ");
    }
    Tensor r(ShapeTag{}, a.sizes(), DType::kBool, DeviceType::kAMD, false);
    uint8_t* out = static_cast<uint8_t*>(r.raw_ptr());
    run(b ? ctamd_compare_f32(cmp, a.fptr(), b->fptr(), out, a.numel(), current_stream())
          : ctamd_compare_scalar_f32(cmp, a.fptr(), s, out, a.numel(), current_stream()),
        "comparison");
    return r;
}
Tensor sum_all(const Tensor& a) {
    check_device(a, "sum");
    Tensor r = scalar0d();
    run(ctamd_sum_f32(a.fptr(), r.fptr(), a.numel(), current_stream()), "sum");
    return r;
}
Tensor unary_declared(op which, const Tensor& a, float param) {
    check_device(a, "unary operator");
    if (!a.is_contiguous()) Ctorch_Error::throwException(kP, ErrorType::TENSOR_STATE, "unary operator: a contiguous tensor is needed");
    Tensor r = like(a);
    void* s = current_stream();
    const size_t n = a.numel();
    int rc = CTAMD_EINVAL;
    switch (which) {
        case op::Abs: rc = ctamd_abs_f32(a.fptr(), r.fptr(), n, s); break;
        case op::Exp: rc = ctamd_exp_f32(a.fptr(), r.fptr(), n, s); break;
        case op::Log: rc = ctamd_log_f32(a.fptr(), r.fptr(), n, s); break;
        case op::Sqrt: rc = ctamd_sqrt_f32(a.fptr(), r.fptr(), n, s); break;
        case op::Square: rc = ctamd_square_f32(a.fptr(), r.fptr(), n, s); break;
        case op::Tan: rc = ctamd_tan_f32(a.fptr(), r.fptr(), n, s); break;
        case op::LReLU: rc = ctamd_leaky_relu_f32(a.fptr(), param, r.fptr(), n, s); break;
        default: Ctorch_Error::throwException(kP, ErrorType::UNKNOWN, "unary operator: not one of the declared methods");
    }
    run(rc, "unary operator");
    return r;
}
Tensor unary_declared_backward(op which, const Tensor& v, const Tensor& g, float param) {
    check_device(v, "unary gradient");
    check_device(g, "unary gradient");
    if (v.numel() != g.numel()) Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "unary gradient: sizes differ");
    if (which == op::Exp) return Mul_AMD_kernel(v, g);            // y * g
    if (which == op::Log) return Div_AMD_kernel(g, v);            // g / x
    Tensor r = like(v);
    void* s = current_stream();
    const size_t n = v.numel();
    int rc = CTAMD_EINVAL;
    switch (which) {
        case op::Abs: rc = ctamd_abs_backward_f32(v.fptr(), g.fptr(), r.fptr(), n, s); break;
        case op::Sqrt: rc = ctamd_sqrt_backward_f32(v.fptr(), g.fptr(), r.fptr(), n, s); break;
        case op::Square: rc = ctamd_square_backward_f32(v.fptr(), g.fptr(), r.fptr(), n, s); break;
        case op::Tan: rc = ctamd_tan_backward_f32(v.fptr(), g.fptr(), r.fptr(), n, s); break;
        case op::LReLU: rc = ctamd_leaky_relu_backward_f32(v.fptr(), g.fptr(), param, r.fptr(), n, s); break;
        default: Ctorch_Error::throwException(kP, ErrorType::UNKNOWN, "unary gradient: not one of the declared methods");
    }
    run(rc, "unary gradient");
    return r;
}
Tensor reduce_axis(int kind, const Tensor& a, size_t outer, size_t len, size_t inner, int ddof,
                   const std::vector<size_t>& result_shape, Tensor* index, Tensor* mean) {
    check_device(a, "reduction");
    if (!a.is_contiguous()) Ctorch_Error::throwException(kP, ErrorType::TENSOR_STATE, "reduction: a contiguous tensor is needed");
    if (len == 0) Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "reduction over an empty dimension");
    Tensor r(ShapeTag{}, result_shape, DType::kFloat, DeviceType::kAMD, false);
    const bool extreme = kind == CTAMD_RED_MAX || kind == CTAMD_RED_MIN, spread = kind == CTAMD_RED_VAR || kind == CTAMD_RED_STD;
    if (index && extreme) *index = Tensor(ShapeTag{}, result_shape, DType::kInt, DeviceType::kAMD, false);
    if (mean && spread) *mean = Tensor(ShapeTag{}, result_shape, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_reduce_dim_f32(kind, a.fptr(), r.fptr(), (index && extreme) ? static_cast<int32_t*>(index->raw_ptr()) : nullptr,
                             (mean && spread) ? mean->fptr() : nullptr, outer, len, inner, ddof, current_stream()),
        "reduction");
    return r;
}
Tensor reduce_axis_backward(int kind, const Tensor& x, const Tensor& y, const Tensor& index, const Tensor& mean, const Tensor& g,
                            size_t outer, size_t len, size_t inner, int ddof) {
    check_device(x, "reduction gradient");
    check_device(g, "reduction gradient");
    if (g.numel() != outer * inner || !g.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "reduction gradient: the upstream gradient does not have the result's size");
    Tensor r = like(x);
    run(ctamd_reduce_dim_backward_f32(kind, x.fptr(), y.is_cleared() ? nullptr : y.fptr(),
                                      index.is_cleared() ? nullptr : static_cast<const int32_t*>(index.raw_ptr()),
                                      mean.is_cleared() ? nullptr : mean.fptr(), g.fptr(), r.fptr(), outer, len, inner, ddof, current_stream()),
        "reduction gradient");
    return r;
}
Tensor log_softmax_dim(const Tensor& a, int dim) {
    check_device(a, "log_softmax");
    if (!a.is_contiguous()) Ctorch_Error::throwException(kP, ErrorType::TENSOR_STATE, "log_softmax: a contiguous tensor is needed");
    Tensor r = like(a);
    size_t rows, cols;
    rows_cols(a, rows, cols);
    if (a.dim() == 1 || dim == 1) run(ctamd_log_softmax_rows_f32(a.fptr(), r.fptr(), rows, cols, current_stream()), "log_softmax");
    else run(ctamd_log_softmax_cols_f32(a.fptr(), r.fptr(), rows, cols, current_stream()), "log_softmax");
    return r;
}
Tensor log_softmax_backward(const Tensor& y, const Tensor& g, int dim) {
    check_device(y, "log_softmax_backward");
    check_device(g, "log_softmax_backward");
    Tensor r = like(y);
    size_t rows, cols;
    rows_cols(y, rows, cols);
    if (y.dim() == 1 || dim == 1) run(ctamd_log_softmax_backward_rows_f32(y.fptr(), g.fptr(), r.fptr(), rows, cols, current_stream()), "log_softmax_backward");
    else run(ctamd_log_softmax_backward_cols_f32(y.fptr(), g.fptr(), r.fptr(), rows, cols, current_stream()), "log_softmax_backward");
    return r;
}
Tensor fold_mod(const Tensor& g, const std::vector<size_t>& target_shape) {
    check_device(g, "fold_mod");
    Tensor r(ShapeTag{}, target_shape, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_fold_mod_f32(g.fptr(), r.fptr(), g.numel(), r.numel(), current_stream()), "fold_mod");
    return r;
}
Tensor broadcast_reduce(const Tensor& g, const std::vector<size_t>& g_shape, const std::vector<size_t>& t_shape,
                        const std::vector<size_t>& result_shape) {
    check_device(g, "broadcast_reduce");
    Tensor r(ShapeTag{}, result_shape, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_broadcast_reduce_f32(g.fptr(), g_shape.data(), t_shape.data(), int(g_shape.size()), r.fptr(), current_stream()), "broadcast_reduce");
    return r;
}
Tensor leading_elements(const Tensor& g, const std::vector<size_t>& shape) {
    check_device(g, "leading_elements");
    Tensor r(ShapeTag{}, shape, DType::kFloat, DeviceType::kAMD, false);
    if (r.numel() > g.numel()) Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "leading_elements: the gradient is too short");
    device_copy_d2d(r.fptr(), g.fptr(), r.numel() * sizeof(float));
    return r;
}
Tensor softmax_dim(const Tensor& a, int dim) {
    if (a.dtype() == DType::kDouble) {                                  // src/Tensor.cpp:1686-1696, :1747-1783
        check_on_device(a, "softmax");
        Tensor r(ShapeTag{}, a.sizes(), DType::kDouble, DeviceType::kAMD, false);
        size_t rows = a.dim() == 1 ? 1 : a.sizes()[0], cols = a.dim() == 1 ? a.sizes()[0] : a.sizes()[1];
        run(ctamd_softmax_f64(static_cast<const double*>(a.raw_ptr()), static_cast<double*>(r.raw_ptr()), rows, cols,
                              a.dim() == 1 ? 1 : dim, current_stream()),
            "softmax");
        return r;
    }
    check_device(a, "softmax");
    Tensor r = like(a);
    size_t rows, cols;
    rows_cols(a, rows, cols);
    if (a.dim() == 1 || dim == 1) run(ctamd_softmax_rows_f32(a.fptr(), r.fptr(), rows, cols, current_stream()), "softmax");
    else run(ctamd_softmax_cols_f32(a.fptr(), r.fptr(), rows, cols, current_stream()), "softmax");
    return r;
}
Tensor filled(const std::vector<size_t>& shape, float v, DeviceType device) {
    Tensor r(ShapeTag{}, shape, DType::kFloat, device, false);
    if (device == DeviceType::kAMD) run(ctamd_fill_f32(r.fptr(), v, r.numel(), current_stream()), "fill");
    else for (size_t i = 0; i < r.numel(); ++i) r.data<float>()[i] = v;
    return r;
}
void fill_scalar(Tensor& t, float v) {
    check_device(t, "fill");
    run(ctamd_fill_f32(t.fptr(), v, t.numel(), current_stream()), "fill");
}
Tensor filled_from(const std::vector<size_t>& shape, const Tensor& s) {
    check_device(s, "fill");
    Tensor r(ShapeTag{}, shape, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_fill_from_f32(r.fptr(), s.fptr(), r.numel(), current_stream()), "fill");
    return r;
}
void accumulate(Tensor& grad, const Tensor& val) {
    check_device(grad, "accumulate");
    check_device(val, "accumulate");
    if (grad.numel() != val.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "accumulate: gradient sizes differ");
    run(ctamd_accumulate_f32(grad.fptr(), val.fptr(), grad.numel(), current_stream()), "accumulate");
    grad.forget_known_value();      // written in place: whatever the host knew of it is gone
}
// grad = 0 + val in one pass: what the reference's "zero-filled gradient, then grad[i] += val[i]"
// (src/AutoDiff.cpp:1870-1907) leaves after the first contribution, bit for bit (-0 becomes +0).
Tensor zero_plus(const Tensor& val, const std::vector<size_t>& shape) {
    check_device(val, "accumulate");
    Tensor r(ShapeTag{}, shape, DType::kFloat, DeviceType::kAMD, false);
    if (r.numel() != val.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "accumulate: gradient sizes differ");
    run(ctamd_add_scalar_f32(val.fptr(), 0.0f, r.fptr(), r.numel(), current_stream()), "accumulate");
    return r;
}
Tensor sum_of(const Tensor& a, const Tensor& b) {
    check_device(a, "accumulate");
    check_device(b, "accumulate");
    if (a.numel() != b.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "accumulate: gradient sizes differ");
    Tensor r = like(a);
    run(ctamd_add_f32(a.fptr(), b.fptr(), r.fptr(), r.numel(), current_stream()), "accumulate");
    return r;
}
Tensor column_sum(const Tensor& g) {
    check_device(g, "column_sum");
    Tensor r(ShapeTag{}, {g.sizes()[1]}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_colsum_f32(g.fptr(), r.fptr(), g.sizes()[0], g.sizes()[1], current_stream()), "column_sum");
    return r;
}
Tensor first_row(const Tensor& g) {
    check_device(g, "first_row");
    Tensor r(ShapeTag{}, {g.sizes()[1]}, DType::kFloat, DeviceType::kAMD, false);
    device_copy_d2d(r.fptr(), g.fptr(), g.sizes()[1] * sizeof(float));
    return r;
}
bool any_abs_lt_eps(const Tensor& b) {
    check_device(b, "any_abs_lt_eps");
    Tensor flag(ShapeTag{}, {}, DType::kFloat, DeviceType::kAMD, false);   // 4 bytes, read as int32
    run(ctamd_any_abs_lt_eps_f32(b.fptr(), reinterpret_cast<int32_t*>(flag.fptr()), b.numel(), current_stream()), "any_abs_lt_eps");
    int32_t v = 0;
    device_copy_d2h(&v, flag.fptr(), sizeof(v));
    return v != 0;
}

void copy_into(Tensor& dst, const Tensor& src) {
    check_device(dst, "copy_into");
    check_device(src, "copy_into");
    if (dst.numel() != src.numel() || !dst.is_contiguous() || !src.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "copy_into: sizes differ or a tensor is not contiguous");
    dst.require_writable("copy_into");
    dst.forget_known_value();
    device_copy_d2d(dst.fptr(), src.fptr(), dst.numel() * sizeof(float));
}
Tensor onehot(const Tensor& labels, size_t classes) {
    check_device(labels, "onehot");
    Tensor r(ShapeTag{}, {labels.numel(), classes}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_onehot_f32(labels.fptr(), r.fptr(), labels.numel(), classes, current_stream()), "onehot");
    return r;
}
void sgd_step(Tensor& param, const Tensor& grad, float lr) {
    check_device(param, "sgd_step");
    check_device(grad, "sgd_step");
    if (param.numel() != grad.numel() || !param.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "sgd_step: parameter and gradient differ in size");
    param.require_writable("sgd_step");
    param.forget_known_value();     // written in place
    run(ctamd_sgd_step_f32(param.fptr(), grad.fptr(), lr, param.numel(), current_stream()), "sgd_step");
}
void sgd_step_all(const std::vector<Tensor*>& params, const std::vector<Tensor>& grads, float lr) {
    if (params.size() != grads.size())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "sgd_step_all: one gradient per parameter");
    std::vector<float*> p;
    std::vector<const float*> g;
    std::vector<size_t> n;
    for (size_t i = 0; i < params.size(); ++i) {
        if (grads[i].is_cleared()) continue;                 // no gradient: p - 0 * lr = p
        check_device(*params[i], "sgd_step_all");
        check_device(grads[i], "sgd_step_all");
        if (params[i]->numel() != grads[i].numel() || !params[i]->is_contiguous() || !grads[i].is_contiguous())
            Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "sgd_step_all: parameter and gradient differ in size");
        params[i]->require_writable("sgd_step_all");
        params[i]->forget_known_value();                     // written in place
        p.push_back(params[i]->fptr());
        g.push_back(grads[i].fptr());
        n.push_back(params[i]->numel());
    }
    run(ctamd_sgd_step_multi_f32(p.data(), g.data(), n.data(), int(p.size()), lr, current_stream()), "sgd_step_all");
}
size_t count_correct(const Tensor& pred, const Tensor& labels) {
    check_device(pred, "count_correct");
    check_device(labels, "count_correct");
    if (pred.dim() != 2 || labels.numel() != pred.sizes()[0])
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "count_correct: predictions must be [rows, classes]");
    Tensor count(ShapeTag{}, {}, DType::kFloat, DeviceType::kAMD, false);   // 4 bytes, used as int32
    run(ctamd_count_correct_f32(pred.fptr(), labels.fptr(), reinterpret_cast<int32_t*>(count.fptr()), pred.sizes()[0],
                                pred.sizes()[1], current_stream()), "count_correct");
    int32_t v = 0;
    device_copy_d2h(&v, count.fptr(), sizeof(v));
    return static_cast<size_t>(v);
}
Tensor unit_from_bytes(const unsigned char* host_bytes, size_t rows, size_t cols) {
    const size_t n = rows * cols;
    Tensor r(ShapeTag{}, {rows, cols}, DType::kFloat, DeviceType::kAMD, false);
    if (n == 0) return r;
    void* staging = device_acquire(n);
    device_copy_h2d(staging, host_bytes, n);
    int rc = ctamd_u8_to_unit_f32(static_cast<const uint8_t*>(staging), r.fptr(), n, current_stream());
    if (rc == CTAMD_OK) rc = ctamd_sync(current_stream());      // the staging block goes back to the pool now
    device_release(staging, n);
    run(rc, "unit_from_bytes");
    return r;
}

namespace {
Tensor grad2(int (*fn)(const float*, const float*, float*, size_t, void*), const char* name, const Tensor& x,
             const Tensor& g) {
    check_device(x, name);
    check_device(g, name);
    if (x.numel() != g.numel()) Ctorch_Error::throwException(kP, ErrorType::DIMENSION, std::string(name) + ": sizes differ");
    Tensor r = like(x);
    run(fn(x.fptr(), g.fptr(), r.fptr(), x.numel(), current_stream()), name);
    return r;
}
}  // namespace
Tensor relu_backward(const Tensor& x, const Tensor& g) { return grad2(ctamd_relu_backward_f32, "relu_backward", x, g); }
Tensor sigmoid_backward(const Tensor& x, const Tensor& g) { return grad2(ctamd_sigmoid_backward_f32, "sigmoid_backward", x, g); }
Tensor tanh_backward(const Tensor& x, const Tensor& g) { return grad2(ctamd_tanh_backward_f32, "tanh_backward", x, g); }
Tensor sin_backward(const Tensor& x, const Tensor& g) { return grad2(ctamd_sin_backward_f32, "sin_backward", x, g); }
Tensor cos_backward(const Tensor& x, const Tensor& g) { return grad2(ctamd_cos_backward_f32, "cos_backward", x, g); }
Tensor softmax_backward(const Tensor& y, const Tensor& g, int dim) {
    check_device(y, "softmax_backward");
    check_device(g, "softmax_backward");
    Tensor r = like(y);
    size_t rows, cols;
    rows_cols(y, rows, cols);
    if (y.dim() == 1 || dim == 1) run(ctamd_softmax_backward_rows_f32(y.fptr(), g.fptr(), r.fptr(), rows, cols, current_stream()), "softmax_backward");
    else run(ctamd_softmax_backward_cols_f32(y.fptr(), g.fptr(), r.fptr(), rows, cols, current_stream()), "softmax_backward");
    return r;
}
Tensor mse_backward(const Tensor& p, const Tensor& t, const Tensor& g) {
    check_device(p, "mse_backward");
    Tensor r = like(p);
    run(ctamd_mse_backward_f32(p.fptr(), t.fptr(), g.fptr(), r.fptr(), p.numel(), current_stream()), "mse_backward");
    return r;
}
Tensor mae_backward(const Tensor& p, const Tensor& t, const Tensor& g) {
    check_device(p, "mae_backward");
    Tensor r = like(p);
    run(ctamd_mae_backward_f32(p.fptr(), t.fptr(), g.fptr(), r.fptr(), p.numel(), current_stream()), "mae_backward");
    return r;
}
Tensor unary_backward_plus(op which, const Tensor& x, const Tensor& g, const Tensor& acc) {
    check_device(x, "backward");
    check_device(g, "backward");
    check_device(acc, "backward");
    if (g.numel() != x.numel() || acc.numel() != x.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "backward: sizes differ");
    typedef int (*Fn)(const float*, const float*, const float*, float*, size_t, void*);
    const Fn fn = which == op::ReLU ? ctamd_relu_backward_acc_f32 : which == op::Sigmoid ? ctamd_sigmoid_backward_acc_f32
                : which == op::Tanh ? ctamd_tanh_backward_acc_f32 : which == op::Sin ? ctamd_sin_backward_acc_f32
                                                                                      : ctamd_cos_backward_acc_f32;
    Tensor r = like(x);
    run(fn(x.fptr(), g.fptr(), acc.fptr(), r.fptr(), x.numel(), current_stream()), "backward");
    return r;
}
Tensor mul_plus(const Tensor& a, const Tensor& b, const Tensor& acc) {
    check_device(a, "backward");
    check_device(b, "backward");
    check_device(acc, "backward");
    if (a.numel() != b.numel() || acc.numel() != a.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "backward: sizes differ");
    Tensor r = like(acc);
    run(ctamd_mul_acc_f32(a.fptr(), b.fptr(), acc.fptr(), r.fptr(), a.numel(), current_stream()), "backward");
    return r;
}
Tensor div_plus(const Tensor& g, const Tensor& b, const Tensor& acc) {
    check_device(g, "backward");
    check_device(b, "backward");
    check_device(acc, "backward");
    if (acc.numel() != g.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "backward: sizes differ");
    Tensor r = like(acc);
    if (b.numel() == g.numel())
        run(ctamd_div_acc_f32(g.fptr(), b.fptr(), acc.fptr(), r.fptr(), g.numel(), current_stream()), "backward");
    else
        run(ctamd_div_rowbcast_acc_f32(g.fptr(), b.fptr(), acc.fptr(), r.fptr(), g.sizes()[0], g.sizes()[1], current_stream()), "backward");
    return r;
}
Tensor loss_backward_plus(bool mae, const Tensor& p, const Tensor& t, const Tensor& g, const Tensor& acc) {
    check_device(p, "loss_backward");
    check_device(acc, "loss_backward");
    if (acc.numel() != p.numel() || t.numel() != p.numel())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "loss_backward: sizes differ");
    Tensor r = like(p);
    run(mae ? ctamd_mae_backward_acc_f32(p.fptr(), t.fptr(), g.fptr(), acc.fptr(), r.fptr(), p.numel(), current_stream())
            : ctamd_mse_backward_acc_f32(p.fptr(), t.fptr(), g.fptr(), acc.fptr(), r.fptr(), p.numel(), current_stream()),
        "loss_backward");
    return r;
}
namespace {
// What the class-index CrossEntropy forward leaves for its backward: per-row (max, sum), or - when
// loss and gradient were computed in one pass - the gradient for an upstream gradient of 1.  Keyed
// by the ids of the logits and target tensors (ids are never re-used), a handful of entries,
// oldest out; a kept gradient is handed out once and leaves the table with it.
struct CeStats {
    size_t logits_id = 0, target_id = 0;
    Tensor stats;
    Tensor grad;
};
constexpr int kCeStatsSlots = 4;
thread_local CeStats t_ce_stats[kCeStatsSlots];
thread_local int t_ce_next = 0;
void remember_ce(const Tensor& logits, const Tensor& target, Tensor stats, Tensor grad) {
    CeStats& slot = t_ce_stats[t_ce_next];
    const int mine = t_ce_next;
    t_ce_next = (t_ce_next + 1) % kCeStatsSlots;
    slot.logits_id = logits.id();
    slot.target_id = target.id();
    slot.stats = std::move(stats);
    slot.grad = std::move(grad);
    size_t held = 0;
    for (const CeStats& c : t_ce_stats)
        if (!c.grad.is_cleared()) held += c.grad.numel() * sizeof(float);
    for (int age = 1; age < kCeStatsSlots && held > g_ce_kept_cap; ++age) {      // mine + 1 is the oldest
        CeStats& old = t_ce_stats[(mine + age) % kCeStatsSlots];
        if (old.grad.is_cleared()) continue;
        held -= old.grad.numel() * sizeof(float);
        old = CeStats();                                                       // its backward recomputes from the logits
    }
}
CeStats* recall_ce(const Tensor& logits, const Tensor& target) {
    for (CeStats& c : t_ce_stats)
        if (c.logits_id == logits.id() && c.target_id == target.id() && c.logits_id != 0) return &c;
    return nullptr;
}
// rows the one-pass kernel keeps in registers: 32768 columns with 128-bit accesses, else 8192
bool ce_row_fits(const Tensor& logits) {
    const size_t cols = logits.sizes()[1];
    const bool vec = cols % 4 == 0 && (reinterpret_cast<uintptr_t>(logits.fptr()) & 15u) == 0;
    return cols <= (vec ? size_t(32768) : size_t(8192));
}
}  // namespace

Tensor cross_entropy_backward(const Tensor& x, const Tensor& target, const Tensor& g) {
    check_device(x, "cross_entropy_backward");
    if (x.dim() != 1 && x.dim() != 2)
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "cross_entropy_backward: logits must be 1-D or 2-D");
    size_t rows, cols;
    rows_cols(x, rows, cols);
    if (x.sizes() == target.sizes()) {
        Tensor r = like(x);
        run(ctamd_cross_entropy_backward_onehot_f32(x.fptr(), target.fptr(), g.fptr(), r.fptr(), rows, cols, current_stream()), "cross_entropy_backward");
        return r;
    }
    if (!(target.dim() == 1 && x.dim() == 2 && target.sizes()[0] == rows))
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "cross_entropy_backward: target shape not understood");
    CeStats* kept = recall_ce(x, target);
    if (kept && !kept->grad.is_cleared()) {
        // the forward pass already formed softmax - onehot: for an upstream gradient of 1 (a loss that
        // is the root of backward()) that is the gradient, d * 1.0f being d.  Handed out once.
        Tensor d = std::move(kept->grad);
        kept->grad = Tensor();
        kept->logits_id = 0;
        if (g.known_value() && *g.known_value() == 1.0f) return d;
        kept = nullptr;
    }
    Tensor r = like(x);
    if (kept && !kept->stats.is_cleared())   // with the forward pass's row statistics the backward pass needs no reductions
        run(ctamd_cross_entropy_backward_index_stats_f32(x.fptr(), target.fptr(), kept->stats.fptr(), g.fptr(), r.fptr(), rows, cols,
                                                         current_stream()), "cross_entropy_backward");
    else
        run(ctamd_cross_entropy_backward_index_f32(x.fptr(), target.fptr(), g.fptr(), r.fptr(), rows, cols, current_stream()), "cross_entropy_backward");
    return r;
}
bool linear_ce_head_fits(const Tensor& h, const Tensor& w, const Tensor& bias, const Tensor& labels) {
    auto dev_float = [](const Tensor& t) { return t.device() == DeviceType::kAMD && t.dtype() == DType::kFloat && t.is_contiguous(); };
    if (!dev_float(h) || !dev_float(w) || !dev_float(bias) || !dev_float(labels)) return false;
    if (h.dim() != 2 || w.dim() != 2 || bias.dim() != 1 || labels.dim() != 1) return false;
    if (w.sizes()[0] != h.sizes()[1] || bias.sizes()[0] != w.sizes()[1] || labels.sizes()[0] != h.sizes()[0] || h.sizes()[0] == 0) return false;
    if ((reinterpret_cast<uintptr_t>(h.fptr()) & 15u) != 0) return false;
    return ctamd_linear_ce_head_fits(h.sizes()[1], w.sizes()[1]) != 0;
}
Tensor linear_ce_head(const Tensor& h, const Tensor& w, const Tensor& bias, const Tensor& labels, bool mask_by_h, Tensor* logits,
                      Tensor& dz, Tensor* dh, Tensor& gw, Tensor& gb) {
    const size_t B = h.sizes()[0], H = h.sizes()[1], N = w.sizes()[1];
    const int labels_ok = labels.class_indices_below(N);       // what the host saw when it uploaded them, if it did
    if (labels_ok == 0 && !recording() && !g_ce_deferred_check) {
        Ctorch_Error::log(ErrorLevel::ERROR, kP, ErrorType::TENSOR_STATE, "linear_cross_entropy: class index out of range");
        return Tensor();
    }
    Tensor pair(ShapeTag{}, {2}, DType::kFloat, DeviceType::kAMD, false);      // loss and bad-label flag side by side: one transfer
    Tensor loss = Tensor::view_element(pair, 0);
    if (logits) *logits = Tensor(ShapeTag{}, {B, N}, DType::kFloat, DeviceType::kAMD, false);
    dz = Tensor(ShapeTag{}, {B, N}, DType::kFloat, DeviceType::kAMD, false);
    if (dh) *dh = Tensor(ShapeTag{}, {B, H}, DType::kFloat, DeviceType::kAMD, false);
    gw = Tensor(ShapeTag{}, {H, N}, DType::kFloat, DeviceType::kAMD, false);
    gb = Tensor(ShapeTag{}, {N}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_linear_ce_head_f32(h.fptr(), w.fptr(), bias.fptr(), labels.fptr(), loss.fptr(), reinterpret_cast<int32_t*>(pair.fptr() + 1),
                                 logits ? logits->fptr() : nullptr, dz.fptr(), dh ? dh->fptr() : nullptr, mask_by_h ? 1 : 0, gw.fptr(),
                                 gb.fptr(), B, H, N, current_stream()),
        "linear_cross_entropy");
    if (recording() || g_ce_deferred_check) return loss;     // as CrossEntropy_AMD_kernel: a bad index then shows as a NaN loss
    if (labels_ok == 1) return loss;                          // nothing to wait for: the indices are known to be in range
    struct { float loss; int32_t bad; } got = {0.0f, 0};
    device_copy_d2h(&got, pair.fptr(), sizeof(got));
    if (got.bad) {
        Ctorch_Error::log(ErrorLevel::ERROR, kP, ErrorType::TENSOR_STATE, "linear_cross_entropy: class index out of range");
        return Tensor();
    }
    loss.set_known_value(got.loss);
    return loss;
}
Tensor div_backward_b(const Tensor& a, const Tensor& b, const Tensor& g) {
    check_device(a, "div_backward");
    Tensor r = like(a);
    if (b.numel() == a.numel())
        run(ctamd_div_backward_b_f32(a.fptr(), b.fptr(), g.fptr(), r.fptr(), a.numel(), current_stream()), "div_backward");
    else   // b is a row vector under a [rows, cols]
        run(ctamd_div_backward_b_rowbcast_f32(a.fptr(), b.fptr(), g.fptr(), r.fptr(), a.sizes()[0], a.sizes()[1],
                                              current_stream()), "div_backward");
    return r;
}

}  // namespace ctorch_amd_host

using namespace ctorch_amd_host;

// ----------------------------------------------------------------------- registered kernels
Tensor Add_AMD_kernel(const Tensor& a, const Tensor& b) { return elementwise(kAdd, a, b, false); }
Tensor Sub_AMD_kernel(const Tensor& a, const Tensor& b) { return elementwise(kSub, a, b, true); }
Tensor Mul_AMD_kernel(const Tensor& a, const Tensor& b) { return elementwise(kMul, a, b, true); }
Tensor Div_AMD_kernel(const Tensor& a, const Tensor& b) { return elementwise(kDiv, a, b, false); }

// MatMul_BASIC_kernel.cpp:25-30: 2-D only, inner extents must agree (both throw); operands may be
// strided views (t()).
Tensor MatMul_AMD_kernel(const Tensor& a, const Tensor& b) {
    check_device(a, "MatMul_AMD_kernel");
    check_device(b, "MatMul_AMD_kernel");
    if (a.shape().size() != 2 || b.shape().size() != 2)
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "MatMul_AMD_kernel: only 2-D tensors");
    if (a.shape()[1] != b.shape()[0])
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "MatMul_AMD_kernel: inner dimensions differ");
    size_t m = a.shape()[0], k = a.shape()[1], n = b.shape()[1];
    Tensor r(ShapeTag{}, {m, n}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_matmul_f32(a.fptr(), int64_t(a.strides()[0]), int64_t(a.strides()[1]), b.fptr(), int64_t(b.strides()[0]),
                         int64_t(b.strides()[1]), r.fptr(), int64_t(m), int64_t(n), int64_t(k), current_stream()),
        "MatMul_AMD_kernel");
    return r;
}
Tensor MatMulReluMask_AMD_kernel(const Tensor& a, const Tensor& b, const Tensor& y) {
    check_device(a, "MatMulReluMask_AMD_kernel");
    check_device(b, "MatMulReluMask_AMD_kernel");
    check_device(y, "MatMulReluMask_AMD_kernel");
    if (a.shape().size() != 2 || b.shape().size() != 2 || a.shape()[1] != b.shape()[0])
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "MatMulReluMask_AMD_kernel: not a product of two matrices");
    size_t m = a.shape()[0], k = a.shape()[1], n = b.shape()[1];
    if (y.shape() != std::vector<size_t>{m, n} || !y.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "MatMulReluMask_AMD_kernel: the activation is not a contiguous [m, n]");
    Tensor r(ShapeTag{}, {m, n}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_matmul_relu_mask_f32(a.fptr(), int64_t(a.strides()[0]), int64_t(a.strides()[1]), b.fptr(), int64_t(b.strides()[0]),
                                   int64_t(b.strides()[1]), y.fptr(), r.fptr(), int64_t(m), int64_t(n), int64_t(k), current_stream()),
        "MatMulReluMask_AMD_kernel");
    return r;
}
Tensor MatMulColSum_AMD_kernel(const Tensor& a, const Tensor& b, Tensor& sums) {
    check_device(a, "MatMulColSum_AMD_kernel");
    check_device(b, "MatMulColSum_AMD_kernel");
    if (a.shape().size() != 2 || b.shape().size() != 2 || a.shape()[1] != b.shape()[0])
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "MatMulColSum_AMD_kernel: not a product of two matrices");
    if (!b.is_contiguous())
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "MatMulColSum_AMD_kernel: the second operand is not contiguous");
    size_t m = a.shape()[0], k = a.shape()[1], n = b.shape()[1];
    Tensor r(ShapeTag{}, {m, n}, DType::kFloat, DeviceType::kAMD, false);
    sums = Tensor(ShapeTag{}, {n}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_matmul_colsum_f32(a.fptr(), int64_t(a.strides()[0]), int64_t(a.strides()[1]), b.fptr(), int64_t(b.strides()[0]),
                                int64_t(b.strides()[1]), r.fptr(), sums.fptr(), int64_t(m), int64_t(n), int64_t(k), current_stream()),
        "MatMulColSum_AMD_kernel");
    return r;
}
Tensor Linear_AMD_kernel(const Tensor& x, const Tensor& w, const Tensor& bias, bool relu) {
    check_device(x, "Linear_AMD_kernel");
    check_device(w, "Linear_AMD_kernel");
    check_device(bias, "Linear_AMD_kernel");
    if (x.shape().size() != 2 || w.shape().size() != 2)
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "Linear_AMD_kernel: only 2-D tensors");
    if (x.shape()[1] != w.shape()[0])
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "Linear_AMD_kernel: inner dimensions differ");
    // the bias must be what operator+ accepts as a row vector (Add_BASIC_kernel.cpp:27-34)
    if (bias.shape().size() != 1 || bias.shape()[0] != w.shape()[1])
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "Linear_AMD_kernel: bias is not a row vector of the result");
    size_t m = x.shape()[0], k = x.shape()[1], n = w.shape()[1];
    Tensor r(ShapeTag{}, {m, n}, DType::kFloat, DeviceType::kAMD, false);
    run(ctamd_matmul_bias_f32(x.fptr(), int64_t(x.strides()[0]), int64_t(x.strides()[1]), w.fptr(), int64_t(w.strides()[0]),
                              int64_t(w.strides()[1]), bias.fptr(), relu ? 1 : 0, r.fptr(), int64_t(m), int64_t(n),
                              int64_t(k), current_stream()),
        "Linear_AMD_kernel");
    return r;
}
Tensor Dot_AMD_kernel(const Tensor& a, const Tensor& b) { return reduce2(ctamd_dot_f32, "Dot_AMD_kernel", a, b, false); }
Tensor MSE_AMD_kernel(const Tensor& a, const Tensor& b) { return reduce2(ctamd_mse_f32, "MSE_AMD_kernel", a, b, true); }
Tensor MAE_AMD_kernel(const Tensor& a, const Tensor& b) { return reduce2(ctamd_mae_f32, "MAE_AMD_kernel", a, b, true); }

// CrossEntropy_BASIC_kernel.cpp: one-hot / soft targets of the logits' shape (:41-82) or class
// indices [rows] (:88-120); an unsupported shape or an out-of-range index logs an error and
// returns an empty Tensor (:86, :96-100, :124).  Loss is the SUM over rows.
Tensor CrossEntropy_AMD_kernel(const Tensor& a, const Tensor& b) {
    check_device(a, "CrossEntropy_AMD_kernel");
    check_device(b, "CrossEntropy_AMD_kernel");
    if (a.sizes() == b.sizes()) {
        if (a.dim() != 1 && a.dim() != 2) {
            Ctorch_Error::log(ErrorLevel::ERROR, kP, ErrorType::DIMENSION, "CrossEntropy_AMD_kernel: one-hot targets need 1-D / 2-D logits");
            return Tensor();
        }
        size_t rows, cols;
        rows_cols(a, rows, cols);
        Tensor r = scalar0d();
        run(ctamd_cross_entropy_onehot_f32(a.fptr(), b.fptr(), r.fptr(), rows, cols, current_stream()), "CrossEntropy_AMD_kernel");
        return r;
    }
    if (b.dim() == 1 && a.dim() == 2 && b.sizes()[0] == a.sizes()[0]) {
        // class indices that came from the host were looked at when they were uploaded: a bad one is
        // refused here, before anything is computed (as the reference does), and good ones leave the
        // host nothing to wait for
        const int labels_ok = b.class_indices_below(a.sizes()[1]);
        if (labels_ok == 0 && !recording() && !g_ce_deferred_check) {
            Ctorch_Error::log(ErrorLevel::ERROR, kP, ErrorType::TENSOR_STATE, "CrossEntropy_AMD_kernel: class index out of range");
            return Tensor();
        }
        // loss and bad-index flag side by side: otherwise the host has to wait for the flag (a bad index
        // returns an empty Tensor), so it fetches the loss in the same transfer and item() is free
        Tensor pair(ShapeTag{}, {2}, DType::kFloat, DeviceType::kAMD, false);
        Tensor r = Tensor::view_element(pair, 0);
        if (g_ce_one_pass && AutoDiffContext::current() && a.requires_grad() && ce_row_fits(a) &&
            a.numel() * sizeof(float) <= g_ce_kept_cap) {
            Tensor grad = like(a);
            run(ctamd_cross_entropy_index_fused_f32(a.fptr(), b.fptr(), r.fptr(), reinterpret_cast<int32_t*>(pair.fptr() + 1),
                                                    grad.fptr(), a.sizes()[0], a.sizes()[1], current_stream()),
                "CrossEntropy_AMD_kernel");
            remember_ce(a, b, Tensor(), std::move(grad));
        } else {
            Tensor stats(ShapeTag{}, {a.sizes()[0], 2}, DType::kFloat, DeviceType::kAMD, false);
            run(ctamd_cross_entropy_index_stats_f32(a.fptr(), b.fptr(), r.fptr(), reinterpret_cast<int32_t*>(pair.fptr() + 1),
                                                    stats.fptr(), a.sizes()[0], a.sizes()[1], current_stream()),
                "CrossEntropy_AMD_kernel");
            remember_ce(a, b, std::move(stats), Tensor());
        }
        // a recorded step cannot wait, and a caller may choose not to (set_ce_deferred_label_check): a
        // bad index then shows as a NaN loss when the loss is read, and the step keeps the GPU busy
        // between its forward and backward passes instead of idling it for the flag's round trip
        if (recording() || g_ce_deferred_check || labels_ok == 1) return r;
        struct { float loss; int32_t bad; } got = {0.0f, 0};
        device_copy_d2h(&got, pair.fptr(), sizeof(got));
        if (got.bad) {
            Ctorch_Error::log(ErrorLevel::ERROR, kP, ErrorType::TENSOR_STATE, "CrossEntropy_AMD_kernel: class index out of range");
            return Tensor();
        }
        r.set_known_value(got.loss);
        return r;
    }
    Ctorch_Error::log(ErrorLevel::ERROR, kP, ErrorType::DIMENSION, "CrossEntropy_AMD_kernel: incompatible shapes");
    return Tensor();
}

Tensor Neg_AMD_kernel(const Tensor& a) { return map(ctamd_neg_f32, "Neg_AMD_kernel", a); }
Tensor ReLU_AMD_kernel(const Tensor& a) { return map(ctamd_relu_f32, "ReLU_AMD_kernel", a); }
Tensor Cos_AMD_kernel(const Tensor& a) { return map(ctamd_cos_f32, "Cos_AMD_kernel", a); }
Tensor Sin_AMD_kernel(const Tensor& a) { return map(ctamd_sin_f32, "Sin_AMD_kernel", a); }
Tensor Tanh_AMD_kernel(const Tensor& a) { return map(ctamd_tanh_f32, "Tanh_AMD_kernel", a); }
Tensor Sigmoid_AMD_kernel(const Tensor& a) { return map(ctamd_sigmoid_f32, "Sigmoid_AMD_kernel", a); }
Tensor LReLU_AMD_kernel(const Tensor& a) { return unary_declared(op::LReLU, a, 0.01f); }
// Softmax_BASIC_kernel.cpp:26-35, :95-98: float only, 1-D or 2-D (last dimension), throws otherwise
Tensor Softmax_AMD_kernel(const Tensor& a) {
    check_device(a, "Softmax_AMD_kernel");
    if (a.dim() != 1 && a.dim() != 2)
        Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "Softmax_AMD_kernel: only 1-D / 2-D tensors");
    return softmax_dim(a, int(a.dim()) - 1);
}
