// Tensor front-end: metadata, transfers and the operator methods.  Each operator method keeps the
// reference's structure (e.g. src/Tensor.cpp:724-747 for operator*): dtype / device checks that
// throw, dispatch through Ctorch_Scheduler, then the two-phase tape record.
#include "Tensor.h"

#include <cfloat>
#include <cmath>
#include <cstring>

#include <algorithm>

#include "Ctorch_Scheduler.h"
#include "ctorch_amd.h"
#include "kernels.h"

using namespace ctorch_amd_host;

std::atomic<size_t> Tensor::global_tensor_id{1};

void Tensor::computeStrides() {
    _strides.assign(_shape.size(), 1);
    for (int i = int(_shape.size()) - 2; i >= 0; --i) _strides[i] = _strides[i + 1] * _shape[i + 1];
}

Tensor::Tensor() : tensor_id_(global_tensor_id++) { computeStrides(); }

Tensor::Tensor(float value) : tensor_id_(global_tensor_id++), _storage(&value, 1, DType::kFloat, DeviceType::kCPU) {
    computeStrides();
}

// On the device the value is written by a one-element fill launch: a host-to-device copy would
// drain the stream first (every `tensor + 5.0f` and every backward() makes one of these).
Tensor::Tensor(float value, DeviceType device)
    : tensor_id_(global_tensor_id++), _device(device),
      _storage(device == DeviceType::kAMD ? Storage(1, DType::kFloat, device) : Storage(&value, 1, DType::kFloat, device)) {
    computeStrides();
    if (device == DeviceType::kAMD) {
        fill_scalar(*this, value);
        set_known_value(value);      // the host just chose it
    }
}

Tensor::Tensor(std::initializer_list<float> values)
    : tensor_id_(global_tensor_id++), _shape({values.size()}), _storage(values.begin(), values.size(), DType::kFloat) {
    computeStrides();
}

Tensor::Tensor(ShapeTag, const std::vector<size_t>& shape, DType dtype, DeviceType device, bool zero_init)
    : tensor_id_(global_tensor_id++), _shape(shape), _device(device), _dtype(dtype) {
    computeStrides();
    _storage = Storage(numel(), dtype, device);
    if (zero_init) zero();
}

Tensor::Tensor(const Tensor& other)
    : tensor_id_(global_tensor_id++), _requires_grad(other._requires_grad), _shape(other._shape),
      _strides(other._strides), _storage_offset(other._storage_offset), _device(other._device),
      _dtype(other._dtype), _storage(other._storage.clone()) {}

Tensor& Tensor::operator=(const Tensor& other) {
    if (this != &other) {
        tensor_id_ = global_tensor_id++;
        _requires_grad = other._requires_grad;
        _shape = other._shape;
        _strides = other._strides;
        _storage_offset = other._storage_offset;
        _device = other._device;
        _dtype = other._dtype;
        _storage = other._storage.clone();
    }
    return *this;
}

Tensor::Tensor(Tensor&& other) noexcept
    : tensor_id_(other.tensor_id_), _requires_grad(other._requires_grad), _shape(std::move(other._shape)),
      _strides(std::move(other._strides)), _storage_offset(other._storage_offset), _device(other._device),
      _dtype(other._dtype), _storage(std::move(other._storage)) {
    other.tensor_id_ = 0;
}

Tensor& Tensor::operator=(Tensor&& other) noexcept {
    if (this != &other) {
        tensor_id_ = other.tensor_id_;
        _requires_grad = other._requires_grad;
        _shape = std::move(other._shape);
        _strides = std::move(other._strides);
        _storage_offset = other._storage_offset;
        _device = other._device;
        _dtype = other._dtype;
        _storage = std::move(other._storage);
        other.tensor_id_ = 0;
    }
    return *this;
}

Tensor::Tensor(AliasTag, const Tensor& other)
    : tensor_id_(other.tensor_id_), _requires_grad(other._requires_grad), _shape(other._shape),
      _strides(other._strides), _storage_offset(other._storage_offset), _device(other._device),
      _dtype(other._dtype), _storage(other._storage) {}

Tensor Tensor::from_host(const float* data, const std::vector<size_t>& shape, DeviceType device) {
    Tensor t(ShapeTag{}, shape, DType::kFloat, device, false);
    if (t.numel()) {
        if (device == DeviceType::kAMD) {
            device_copy_h2d(t.fptr(), data, t.numel() * sizeof(float));
            t._storage.note_uploaded_floats(data, t.numel());
        } else {
            std::memcpy(t.data<float>(), data, t.numel() * sizeof(float));
        }
    }
    return t;
}

size_t Tensor::numel() const {
    if (_shape.empty()) return 1;
    return std::accumulate(_shape.begin(), _shape.end(), size_t(1), std::multiplies<size_t>());
}

bool Tensor::is_contiguous() const {
    size_t expect = 1;
    for (int i = int(_shape.size()) - 1; i >= 0; --i) {
        if (_shape[i] != 1 && _strides[i] != expect) return false;
        expect *= _shape[i];
    }
    return true;
}

void Tensor::requires_grad(bool key) {
    _requires_grad = key;
    if (key && AutoDiffContext::current()) {
        AutoDiffContext::current()->make_leaf(*this, key);
        AutoDiffContext::current()->update_requires_grad(*this, key);
    }
}

template <>
float Tensor::item<float>() const {
    if (numel() != 1 || _storage.empty())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "item(): tensor is not a single element");
    if (_dtype != DType::kFloat)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "item<float>(): dtype is not float");
    if (_device == DeviceType::kAMD) {
        if (const float* v = known_value()) return *v;
        float v;
        device_copy_d2h(&v, fptr(), sizeof(float));
        return v;
    }
    return *data<float>();
}

std::vector<float> Tensor::to_vector() const {
    std::vector<float> out(numel());
    if (out.empty() || _storage.empty()) return out;
    if (_dtype != DType::kFloat)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "to_vector(): dtype is not float");
    if (is_contiguous()) {
        if (_device == DeviceType::kAMD) device_copy_d2h(out.data(), fptr(), out.size() * sizeof(float));
        else std::memcpy(out.data(), data<float>(), out.size() * sizeof(float));
        return out;
    }
    // strided view: bring the whole storage over and gather
    std::vector<float> all(_storage.size());
    if (_device == DeviceType::kAMD) device_copy_d2h(all.data(), _storage.raw(), all.size() * sizeof(float));
    else std::memcpy(all.data(), _storage.raw(), all.size() * sizeof(float));
    std::vector<size_t> idx(_shape.size(), 0);
    for (size_t n = 0; n < out.size(); ++n) {
        size_t off = _storage_offset;
        for (size_t d = 0; d < idx.size(); ++d) off += idx[d] * _strides[d];
        out[n] = all[off];
        for (int d = int(idx.size()) - 1; d >= 0; --d) {
            if (++idx[d] < _shape[d]) break;
            idx[d] = 0;
        }
    }
    return out;
}

Tensor Tensor::to(DeviceType device) const {
    Tensor r(AliasTag{}, *this);
    r.tensor_id_ = global_tensor_id++;
    r._storage = _storage.to(device);
    r._device = device;
    return r;
}

void Tensor::fill(float v) {
    require_writable("fill");
    forget_known_value();
    if (_storage.empty()) return;
    if (_dtype != DType::kFloat)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "fill(): only float tensors");
    if (_device == DeviceType::kAMD) {
        Tensor f = filled({_storage.size()}, v, DeviceType::kAMD);
        device_copy_d2d(_storage.raw(), f.fptr(), _storage.nbytes());
    } else {
        float* p = _storage.data<float>();
        for (size_t i = 0; i < _storage.size(); ++i) p[i] = v;
    }
}
// src/Tensor.cpp:390-448: every dtype, the whole storage
void Tensor::zero() {
    if (_storage.empty()) return;
    if (_dtype == DType::kFloat) { fill(0.0f); return; }
    if (_device == DeviceType::kAMD) { ctorch_amd_host::fill_typed(_storage.raw(), _dtype, 0.0, _storage.size()); return; }
    std::memset(_storage.raw(), 0, _storage.nbytes());
}
void Tensor::ones() {
    if (_storage.empty()) return;
    if (_dtype == DType::kFloat) { fill(1.0f); return; }
    if (_device == DeviceType::kAMD) { ctorch_amd_host::fill_typed(_storage.raw(), _dtype, 1.0, _storage.size()); return; }
    const size_t n = _storage.size();
    switch (_dtype) {
        case DType::kDouble: for (size_t i = 0; i < n; ++i) _storage.data<double>()[i] = 1.0; break;
        case DType::kInt: for (size_t i = 0; i < n; ++i) _storage.data<int32_t>()[i] = 1; break;
        case DType::kLong: for (size_t i = 0; i < n; ++i) _storage.data<int64_t>()[i] = 1; break;
        default: std::memset(_storage.raw(), 1, _storage.nbytes());
    }
}

Tensor Tensor::to(DType dtype) const {
    if (_dtype == dtype) return *this;
    if (_dtype != DType::kFloat)    // the reference returns an uninitialised tensor here (src/Tensor.cpp:206: only float sources are converted)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "to(dtype): only float tensors are converted");
    if (_device != DeviceType::kAMD)
        Ctorch_Error::throwException(ErrorPlatform::kCPU, ErrorType::DEVICE_COMPAT, "to(dtype): computed on the AMD device only");
    return ctorch_amd_host::cast_from_float(*this, dtype);
}

Tensor Tensor::transpose(int dim0, int dim1) const {
    if (dim0 < 0 || dim0 >= int(_shape.size()) || dim1 < 0 || dim1 >= int(_shape.size()))
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DIMENSION, "transpose: dimension out of range");
    Tensor result(*this);
    std::swap(result._shape[dim0], result._shape[dim1]);
    std::swap(result._strides[dim0], result._strides[dim1]);
    return result;
}
Tensor Tensor::t() const { return transpose(0, 1); }

Tensor Tensor::view_t(const Tensor& t) {
    if (t._shape.size() != 2)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DIMENSION, "view_t: tensor is not 2-D");
    Tensor r(AliasTag{}, t);
    r.tensor_id_ = global_tensor_id++;
    std::swap(r._shape[0], r._shape[1]);
    std::swap(r._strides[0], r._strides[1]);
    return r;
}

Tensor Tensor::share(const Tensor& t) {
    Tensor r(AliasTag{}, t);
    r.tensor_id_ = global_tensor_id++;
    r._requires_grad = false;
    r._storage.freeze();
    return r;
}

void Tensor::require_writable(const char* what) {
    if (!_storage.writable())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE,
                                     std::string(what) + ": this tensor shares a gradient's bytes with the tape (grad() does not copy); "
                                     "copy it before writing to it in place");
}

Tensor Tensor::view_rows(const Tensor& t, size_t first, size_t count) {
    if (t._shape.empty() || !t.is_contiguous() || first + count > t._shape[0])
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DIMENSION, "view_rows: rows out of range or tensor not contiguous");
    Tensor r(AliasTag{}, t);
    r.tensor_id_ = global_tensor_id++;
    r._requires_grad = false;
    r._storage_offset = t._storage_offset + first * t._strides[0];
    r._shape[0] = count;
    return r;
}

Tensor Tensor::view_element(const Tensor& t, size_t index) {
    if (!t.is_contiguous() || index >= t.numel())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DIMENSION, "view_element: index out of range or tensor not contiguous");
    Tensor r(AliasTag{}, t);
    r.tensor_id_ = global_tensor_id++;
    r._requires_grad = false;
    r._storage_offset = t._storage_offset + index;
    r._shape.clear();
    r.computeStrides();
    return r;
}

Tensor Tensor::view_shape(const Tensor& t, const std::vector<size_t>& shape) {
    size_t n = 1;
    for (size_t e : shape) n *= e;
    if (!t.is_contiguous() || n != t.numel())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DIMENSION, "view_shape: element counts differ or tensor not contiguous");
    Tensor r(AliasTag{}, t);
    r.tensor_id_ = global_tensor_id++;
    r._requires_grad = false;
    r._shape = shape;
    r.computeStrides();
    return r;
}

Tensor Tensor::contiguous() const {
    if (is_contiguous()) return Tensor(*this);
    std::vector<float> v = to_vector();
    Tensor r = from_host(v.data(), _shape, _device);
    r._requires_grad = _requires_grad;
    return r;
}

// ------------------------------------------------------------------------------- operators
namespace {

void check_pair(const Tensor& a, const Tensor& b) {
    if (a.dtype() != b.dtype())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "tensor dtypes differ");
    if (a.device() != b.device())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DEVICE_COMPAT, "tensors are on different devices");
}

// defer_record + commit_record, as every operator method of the reference does
void tape(Tensor& result, op o, std::initializer_list<const Tensor*> inputs, int param = 0,
          std::shared_ptr<AutoDiff::OpPayload> payload = nullptr) {
    AutoDiff* ctx = AutoDiffContext::current();
    if (!ctx) return;
    std::vector<Tensor*> in;
    bool rg = false;
    for (const Tensor* t : inputs) {
        in.push_back(const_cast<Tensor*>(t));
        rg = rg || t->requires_grad();
    }
    ctx->defer_record(result.id(), o, in, param, std::move(payload));
    result.set_requires_grad(rg);
    if (rg) ctx->commit_record(result);
}

Tensor binary(const Tensor& a, const Tensor& b, op o) {
    check_pair(a, b);
    Tensor result = Ctorch_Scheduler::getInstance().dispatch(a, b, o);
    tape(result, o, {&a, &b});
    return result;
}
Tensor unary(const Tensor& a, op o) {
    Tensor result = Ctorch_Scheduler::getInstance().dispatch(a, o);
    tape(result, o, {&a});
    return result;
}

}  // namespace

Tensor Tensor::operator+(const Tensor& other) const { return binary(*this, other, op::Add); }
Tensor Tensor::operator-(const Tensor& other) const { return binary(*this, other, op::Sub); }
Tensor Tensor::operator*(const Tensor& other) const { return binary(*this, other, op::Mul); }
Tensor Tensor::operator/(const Tensor& other) const { return binary(*this, other, op::Div); }
Tensor Tensor::matmul(const Tensor& other) const { return binary(*this, other, op::MatMul); }
Tensor Tensor::linear(const Tensor& weight, const Tensor& bias, bool relu) const {
    if (device() != DeviceType::kAMD) {
        Tensor z = matmul(weight) + bias;
        return relu ? z.relu() : z;
    }
    check_pair(*this, weight);
    check_pair(*this, bias);
    Tensor result = Linear_AMD_kernel(*this, weight, bias, relu);
    tape(result, op::Linear, {this, &weight, &bias}, relu ? 1 : 0);
    return result;
}
Tensor Tensor::linear_cross_entropy(const Tensor& weight, const Tensor& bias, const Tensor& labels, Tensor* logits) const {
    if (!ctorch_amd_host::linear_ce_head_fits(*this, weight, bias, labels)) {
        Tensor z = linear(weight, bias, false);
        if (logits) *logits = Tensor::alias(z);
        return z.cross_entropy(labels);
    }
    AutoDiff* ctx = AutoDiffContext::current();
    const bool taped = ctx && (requires_grad() || weight.requires_grad() || bias.requires_grad());
    auto kept = std::make_shared<AutoDiff::LinearCEPayload>();
    kept->labels = Tensor::alias(labels);
    // under a tape the gradient of x is formed too, at the pre-activation when x comes out of a ReLU layer
    const bool want_dh = taped && requires_grad();
    kept->dh_masked = want_dh && ctx->is_relu_layer_output(*this);
    Tensor result = ctorch_amd_host::linear_ce_head(*this, weight, bias, labels, kept->dh_masked, logits, kept->dz, want_dh ? &kept->dh : nullptr,
                                                    kept->gw, kept->gb);
    if (result.is_cleared()) return result;                       // a class index out of range: logged, empty, as cross_entropy
    if (taped) tape(result, op::LinearCE, {this, &weight, &bias}, 0, kept);
    return result;
}
namespace {
Tensor compare_with(int cmp, const Tensor& a, const Tensor* b, float s) {
    if (a.device() != DeviceType::kAMD)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::PLATFORM_API, "comparison: no kernel for this device");
    return ctorch_amd_host::compare_op(cmp, a, b, s);
}
}  // namespace
Tensor Tensor::operator>(float s) const { return compare_with(CTAMD_CMP_GT, *this, nullptr, s); }
Tensor Tensor::operator<(float s) const { return compare_with(CTAMD_CMP_LT, *this, nullptr, s); }
Tensor Tensor::operator==(float s) const { return compare_with(CTAMD_CMP_EQ, *this, nullptr, s); }
Tensor Tensor::operator>=(float s) const { return compare_with(CTAMD_CMP_GE, *this, nullptr, s); }
Tensor Tensor::operator<=(float s) const { return compare_with(CTAMD_CMP_LE, *this, nullptr, s); }
Tensor Tensor::operator!=(float s) const { return compare_with(CTAMD_CMP_NE, *this, nullptr, s); }
Tensor Tensor::operator>(const Tensor& o) const { return compare_with(CTAMD_CMP_GT, *this, &o, 0.0f); }
Tensor Tensor::operator<(const Tensor& o) const { return compare_with(CTAMD_CMP_LT, *this, &o, 0.0f); }
Tensor Tensor::operator==(const Tensor& o) const { return compare_with(CTAMD_CMP_EQ, *this, &o, 0.0f); }
Tensor Tensor::operator>=(const Tensor& o) const { return compare_with(CTAMD_CMP_GE, *this, &o, 0.0f); }
Tensor Tensor::operator<=(const Tensor& o) const { return compare_with(CTAMD_CMP_LE, *this, &o, 0.0f); }
Tensor Tensor::operator!=(const Tensor& o) const { return compare_with(CTAMD_CMP_NE, *this, &o, 0.0f); }

std::vector<unsigned char> Tensor::to_bytes() const {
    std::vector<unsigned char> out(numel());
    if (out.empty() || _storage.empty()) return out;
    if (!is_contiguous())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "to_bytes(): a contiguous tensor is needed");
    out.resize(numel() * dtypeSize(_dtype));
    const unsigned char* src = static_cast<const unsigned char*>(raw_ptr());
    if (_device == DeviceType::kAMD) device_copy_d2h(out.data(), src, out.size());
    else std::memcpy(out.data(), src, out.size());
    return out;
}

Tensor Tensor::mse_loss(const Tensor& target) const { return binary(*this, target, op::MSE); }
Tensor Tensor::mae_loss(const Tensor& target) const { return binary(*this, target, op::MAE); }
Tensor Tensor::cross_entropy(const Tensor& target) const { return binary(*this, target, op::CE); }
// The reference tapes Dot with its first operand only and has no gradient for it
// (src/Tensor.cpp:593-595, src/AutoDiff.cpp:1856-1862); both operands are taped here and the tape
// has the closed form (an extension).
Tensor Tensor::dot(const Tensor& other) const { return binary(*this, other, op::Dot); }
Tensor Tensor::operator-() const { return unary(*this, op::Neg); }
Tensor Tensor::relu() const { return unary(*this, op::ReLU); }
Tensor Tensor::sigmoid() const { return unary(*this, op::Sigmoid); }
Tensor Tensor::tanh() const { return unary(*this, op::Tanh); }
Tensor Tensor::sin() const { return unary(*this, op::Sin); }
Tensor Tensor::cos() const { return unary(*this, op::Cos); }

namespace {
// tensor (op) float: the reference clones and updates in place on the host, then tapes the op with
// a temporary 0-D tensor as second input (src/Tensor.cpp:794-796, :898-900, :961-963)
Tensor with_scalar(const Tensor& a, float s, op o) {
    Tensor result = scalar_op(a, s, o);
    if (AutoDiffContext::current()) {
        // the taped second input stays on the host: its value is only needed by the gradient of
        // tensor * s and tensor / s, which take it as a launch argument (a device copy of it would
        // cost an allocation and a fill launch per scalar operator)
        Tensor scalar_tensor(s);
        tape(result, o, {&a, &scalar_tensor});
        result.set_requires_grad(a.requires_grad());
    } else {
        result.set_requires_grad(a.requires_grad());
    }
    return result;
}
}  // namespace

Tensor Tensor::operator+(float scalar) const { return with_scalar(*this, scalar, op::Add); }
Tensor Tensor::operator*(float scalar) const { return with_scalar(*this, scalar, op::Mul); }
Tensor Tensor::operator/(float scalar) const {
    if (std::fabs(scalar) < FLT_EPSILON)   // src/Tensor.cpp:919-921
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "division by a (near) zero scalar");
    return with_scalar(*this, scalar, op::Div);
}

Tensor Tensor::sum() const {
    Tensor result = sum_all(*this);
    tape(result, op::Sum, {this});
    return result;
}

Tensor Tensor::softmax(int dim) const {
    if (_shape.empty())
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "softmax: 0-D tensor");
    int rank = int(_shape.size());
    if (dim < 0) dim += rank;
    if (dim < 0 || dim >= rank)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "softmax: dim out of range");
    if (rank > 2)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "softmax: only 1-D / 2-D tensors");
    Tensor result = softmax_dim(*this, dim);
    tape(result, op::Softmax, {this}, dim);
    return result;
}

// ------------------------------------------- declared by the reference, defined only here
namespace {
void need_device(const Tensor& t, const char* what) {
    if (t.device() != DeviceType::kAMD)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::PLATFORM_API, std::string(what) + ": no kernel for this device");
}
Tensor declared_unary(const Tensor& a, op o, float param = 0.0f) {
    need_device(a, "unary operator");
    Tensor result = unary_declared(o, a, param);
    int bits = 0;
    std::memcpy(&bits, &param, sizeof(bits));
    tape(result, o, {&a}, bits);
    return result;
}

// dims -> sorted, unique, non-negative; none = every dimension
std::vector<int> normalised_dims(const Tensor& t, const std::vector<int>& dims) {
    const int rank = int(t.dim());
    std::vector<int> out;
    if (dims.empty()) {
        for (int d = 0; d < rank; ++d) out.push_back(d);
        return out;
    }
    for (int d : dims) {
        if (d < 0) d += rank;
        if (d < 0 || d >= rank)
            Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "reduction: dim out of range");
        out.push_back(d);
    }
    std::sort(out.begin(), out.end());
    out.erase(std::unique(out.begin(), out.end()), out.end());
    return out;
}

// dimensions d0..d1 (adjacent) of `t` reduced in one launch and one tape entry
Tensor reduce_block(const Tensor& t, int kind, int d0, int d1, bool keepdim, int ddof) {
    const std::vector<size_t>& sh = t.shape();
    size_t outer = 1, len = 1, inner = 1;
    std::vector<size_t> result_shape;
    for (int d = 0; d < int(sh.size()); ++d) {
        if (d < d0) outer *= sh[d];
        else if (d <= d1) len *= sh[d];
        else inner *= sh[d];
        if (d < d0 || d > d1) result_shape.push_back(sh[d]);
        else if (keepdim) result_shape.push_back(1);
    }
    const bool taped = AutoDiffContext::current() && t.requires_grad();
    auto payload = std::make_shared<AutoDiff::ReducePayload>();
    payload->kind = kind;
    payload->ddof = ddof;
    payload->outer = outer;
    payload->len = len;
    payload->inner = inner;
    Tensor result = reduce_axis(kind, t, outer, len, inner, ddof, result_shape, taped ? &payload->index : nullptr,
                                taped ? &payload->mean : nullptr);
    tape(result, op::Reduce, {&t}, kind, payload);
    return result;
}

Tensor reduce_dims(const Tensor& t, int kind, const std::vector<int>& dims, bool keepdim, int ddof) {
    need_device(t, "reduction");
    if (t.dtype() != DType::kFloat)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DATATYPE, "reduction: only float32 tensors");
    if (t.dim() == 0) return reduce_block(t, kind, 0, -1, keepdim, ddof);       // one element: len = 1
    const std::vector<int> ds = normalised_dims(t, dims);
    bool adjacent = true;
    for (size_t i = 1; i < ds.size(); ++i) adjacent = adjacent && ds[i] == ds[i - 1] + 1;
    if (adjacent) return reduce_block(t, kind, ds.front(), ds.back(), keepdim, ddof);
    if (kind == CTAMD_RED_VAR || kind == CTAMD_RED_STD)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "var / std: the dimensions must be adjacent");
    // separated dimensions: one after the other from the last, which leaves the earlier ones in place
    Tensor r = reduce_block(t, kind, ds.back(), ds.back(), keepdim, ddof);
    for (size_t i = ds.size() - 1; i-- > 0;) r = reduce_block(r, kind, ds[i], ds[i], keepdim, ddof);
    return r;
}
}  // namespace

Tensor Tensor::operator-(float scalar) const { return with_scalar(*this, scalar, op::Sub); }
Tensor Tensor::abs() const { return declared_unary(*this, op::Abs); }
Tensor Tensor::exp() const { return declared_unary(*this, op::Exp); }
Tensor Tensor::log() const { return declared_unary(*this, op::Log); }
Tensor Tensor::sqrt() const { return declared_unary(*this, op::Sqrt); }
Tensor Tensor::square() const { return declared_unary(*this, op::Square); }
Tensor Tensor::tan() const { return declared_unary(*this, op::Tan); }
Tensor Tensor::leaky_relu(float negative_slope) const {
    if (negative_slope == 0.01f) {
        // the default slope is the registered kernel's (the reference's kernel signature has no room for a slope)
        Tensor result = Ctorch_Scheduler::getInstance().dispatch(*this, op::LReLU);
        int bits = 0;
        std::memcpy(&bits, &negative_slope, sizeof(bits));
        tape(result, op::LReLU, {this}, bits);
        return result;
    }
    return declared_unary(*this, op::LReLU, negative_slope);
}
Tensor Tensor::log_softmax(int dim) const {
    need_device(*this, "log_softmax");
    if (_shape.empty())
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "log_softmax: 0-D tensor");
    int rank = int(_shape.size());
    if (dim < 0) dim += rank;
    if (dim < 0 || dim >= rank)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "log_softmax: dim out of range");
    if (rank > 2)
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::DIMENSION, "log_softmax: only 1-D / 2-D tensors");
    Tensor result = log_softmax_dim(*this, dim);
    tape(result, op::LogSoftmax, {this}, dim);
    return result;
}
Tensor Tensor::sum(const std::vector<int>& dims, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_SUM, dims, keepdim, 0); }
Tensor Tensor::sum(int dim, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_SUM, {dim}, keepdim, 0); }
Tensor Tensor::mean(const std::vector<int>& dims, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_MEAN, dims, keepdim, 0); }
Tensor Tensor::mean(int dim, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_MEAN, {dim}, keepdim, 0); }
Tensor Tensor::mean() const { return reduce_dims(*this, CTAMD_RED_MEAN, {}, false, 0); }
Tensor Tensor::max(const std::vector<int>& dims, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_MAX, dims, keepdim, 0); }
Tensor Tensor::max(int dim, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_MAX, {dim}, keepdim, 0); }
Tensor Tensor::max() const { return reduce_dims(*this, CTAMD_RED_MAX, {}, false, 0); }
Tensor Tensor::min(const std::vector<int>& dims, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_MIN, dims, keepdim, 0); }
Tensor Tensor::min(int dim, bool keepdim) const { return reduce_dims(*this, CTAMD_RED_MIN, {dim}, keepdim, 0); }
Tensor Tensor::min() const { return reduce_dims(*this, CTAMD_RED_MIN, {}, false, 0); }
Tensor Tensor::var_of(const std::vector<int>& dims, bool keepdim, int ddof) const { return reduce_dims(*this, CTAMD_RED_VAR, dims, keepdim, ddof); }
Tensor Tensor::std_of(const std::vector<int>& dims, bool keepdim, int ddof) const { return reduce_dims(*this, CTAMD_RED_STD, dims, keepdim, ddof); }
Tensor Tensor::var(const std::vector<int>& dims, bool keepdim) const { return var_of(dims, keepdim, 1); }
Tensor Tensor::var(int dim, bool keepdim) const { return var_of({dim}, keepdim, 1); }
Tensor Tensor::var() const { return var_of({}, false, 1); }
Tensor Tensor::std(const std::vector<int>& dims, bool keepdim) const { return std_of(dims, keepdim, 1); }
Tensor Tensor::std(int dim, bool keepdim) const { return std_of({dim}, keepdim, 1); }
Tensor Tensor::std() const { return std_of({}, false, 1); }
Tensor Tensor::matmul_unified(const Tensor& other) const { return matmul(other); }

// --------------------------------------------------------------------------------- autograd
void Tensor::backward() const {
    if (!AutoDiffContext::current())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "backward needs an autograd context");
    if (!_requires_grad)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "tensor does not require grad");
    if (is_cleared() || numel() == 0)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "tensor has no data");
    AutoDiffContext::current()->backward(const_cast<Tensor&>(*this));
}
void Tensor::backward(const Tensor& grad_output) const {
    if (!AutoDiffContext::current())
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "backward needs an autograd context");
    if (!_requires_grad)
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "tensor does not require grad");
    AutoDiffContext::current()->backward(const_cast<Tensor&>(*this), Tensor(grad_output));
}

void backward(Tensor& root) {
    if (AutoDiffContext::current()) AutoDiffContext::current()->backward(root);
}
void backward(Tensor& root, Tensor grad_output) {
    if (AutoDiffContext::current()) AutoDiffContext::current()->backward(root, std::move(grad_output));
}
Tensor grad(const Tensor& t) {
    if (AutoDiffContext::current()) return AutoDiffContext::current()->get_grad(&t);
    return Tensor();
}
Tensor matMul(const Tensor& a, const Tensor& b) { return Ctorch_Scheduler::getInstance().dispatch(a, b, op::MatMul); }

bool Ctorch_Scheduler::isDeviceAvailable(DeviceType dev_type) {
    if (dev_type != DeviceType::kAMD) return false;
    try {
        ctorch_amd_host::init_device();
        return true;
    } catch (const std::exception&) {
        return false;
    }
}
