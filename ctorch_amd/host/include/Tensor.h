// Tensor front-end over the MI355X launch layer.  Mirrors the part of the reference's class Tensor
// (include/Tensor.h:70-1123, src/Tensor.cpp) that lies on the operator hot path: construction,
// metadata, the sixteen operator methods that dispatch through Ctorch_Scheduler
// (src/Tensor.cpp:484,574,590,606,622,681,709,736,811,839,1396,1612,1629,1807,1824,1841), the
// host-inline ones (sum :638-666, tensor (op) float :751-973, softmax(dim) :1645-1803,
// transpose / t :246-261, zero / ones :390-451, item :155-165) and backward() / grad().
//
// Semantics kept from the reference: a copy is a deep copy with a new id (Tensor.h:320-334), a
// move keeps the id (:364-377); ids are the tape's keys; results take the first operand's shape;
// ops throw on dtype / device mismatch (src/Tensor.cpp:726-733).
// New: DeviceType::kAMD tensors live in HBM; to(device) / cpu() / amd() are the explicit
// transfers; data<T>() on a device tensor throws; item() copies one element back.
// Arithmetic exists for kAMD tensors only - kCPU tensors are staging containers (the reference's
// CPU kernels are not part of this library), and dispatching one reports "no kernel" loudly.
#ifndef CTORCH_AMD_HOST_TENSOR_H
#define CTORCH_AMD_HOST_TENSOR_H
#include <atomic>
#include <initializer_list>
#include <numeric>
#include <vector>

#include "Ctools.h"
#include "Ctorch_Error.h"
#include "Storage.h"

struct ShapeTag {};

class Tensor {
   private:
    size_t tensor_id_;
    bool _requires_grad = false;
    std::vector<size_t> _shape;
    std::vector<size_t> _strides;
    size_t _storage_offset = 0;
    DeviceType _device = DeviceType::kCPU;
    DType _dtype = DType::kFloat;
    Storage _storage;

    static std::atomic<size_t> global_tensor_id;
    void computeStrides();
    struct AliasTag {};
    Tensor(AliasTag, const Tensor& other);   // shares storage AND id: the tape's reference to a tensor

   public:
    Tensor();
    Tensor(float value);                                         // 0-D tensor on the host
    Tensor(float value, DeviceType device);                      // 0-D tensor on `device`
    Tensor(std::initializer_list<float> values);                 // 1-D host tensor
    Tensor(ShapeTag, const std::vector<size_t>& shape, DType dtype = DType::kFloat,
           DeviceType device = DeviceType::kCPU, bool zero_init = true);
    Tensor(const Tensor& other);                                 // deep copy, new id
    Tensor& operator=(const Tensor& other);
    Tensor(Tensor&& other) noexcept;                             // keeps the id
    Tensor& operator=(Tensor&& other) noexcept;
    ~Tensor() = default;

    static Tensor alias(const Tensor& t) { return Tensor(AliasTag{}, t); }
    // the same bytes as a tensor of its own (new id, not on the tape): read-only sharing
    static Tensor share(const Tensor& t);
    // transposed VIEW of a 2-D tensor: shares storage, no copy (the tape's B^T / A^T operands)
    static Tensor view_t(const Tensor& t);
    // rows [first, first + count) of a contiguous tensor as a VIEW (shares storage, new id): what
    // the demo's get_batch copies out (mnist/mnist.cpp:159-182) without the copy
    static Tensor view_rows(const Tensor& t, size_t first, size_t count);
    // element `index` of a contiguous tensor as a 0-D VIEW (shares storage, new id)
    static Tensor view_element(const Tensor& t, size_t index);
    // the elements of a contiguous tensor under another shape of the same element count, as a VIEW
    // (shares storage, new id)
    static Tensor view_shape(const Tensor& t, const std::vector<size_t>& shape);
    // value of a one-element device tensor when the host already holds it (it chose it, or it came back
    // with another read): item() then needs no transfer.  Kept with the storage, dropped by the in-place writers.
    void set_known_value(float v) { if (numel() == 1) _storage.set_known_value(v); }
    void forget_known_value() { _storage.forget_known_value(); }       // for every tensor that shares the storage
    // throws when this tensor shares a gradient's bytes with the tape (AutoDiff::get_grad): such bytes are read-only
    void require_writable(const char* what);
    const float* known_value() const { return numel() == 1 ? _storage.known_value() : nullptr; }   // null when the host does not know it
    // 1 / 0: the host saw these floats when it uploaded them and, read as class indices, every one lies /
    // some do not lie in [0, classes); -1: it does not know (Storage::class_indices_below)
    int class_indices_below(size_t classes) const { return _storage.class_indices_below(classes); }
    // a tensor on `device` filled from host memory
    static Tensor from_host(const float* data, const std::vector<size_t>& shape, DeviceType device);

    // ---- metadata
    size_t id() const { return tensor_id_; }
    void set_id(size_t id) { tensor_id_ = id; }
    void requires_grad(bool key);
    bool requires_grad() const { return _requires_grad; }
    void set_requires_grad(bool r) { _requires_grad = r; }
    const std::vector<size_t>& shape() const { return _shape; }
    const std::vector<size_t>& sizes() const { return _shape; }
    const std::vector<size_t>& strides() const { return _strides; }
    size_t dim() const { return _shape.size(); }
    size_t numel() const;
    DType dtype() const { return _dtype; }
    DeviceType device() const { return _device; }
    bool is_contiguous() const;
    bool is_cleared() const { return _storage.empty(); }
    const Storage& storage() const { return _storage; }

    // ---- data access
    template <typename T>
    const T* data() const { return _storage.data<T>() + _storage_offset; }   // host tensors only
    template <typename T>
    T* data() { return _storage.data<T>() + _storage_offset; }
    // fp32 pointer in the tensor's own address space (HBM for kAMD), offset applied
    bool storage_shared() const { return _storage.shared(); }
    // first byte of the elements, any dtype (device or host memory, as device() says)
    void* raw_ptr() { return static_cast<char*>(_storage.raw()) + _storage_offset * dtypeSize(_dtype); }
    const void* raw_ptr() const { return static_cast<const char*>(_storage.raw()) + _storage_offset * dtypeSize(_dtype); }
    const float* fptr() const { return static_cast<const float*>(_storage.raw()) + _storage_offset; }
    float* fptr() { return static_cast<float*>(_storage.raw()) + _storage_offset; }
    template <typename T>
    T item() const;
    std::vector<float> to_vector() const;     // contiguous host copy of the elements (any device)

    // ---- transfers
    Tensor to(DeviceType device) const;
    Tensor to(DType dtype) const;            // from float only, as src/Tensor.cpp:197-243
    Tensor cpu() const { return to(DeviceType::kCPU); }
    Tensor amd() const { return to(DeviceType::kAMD); }

    // ---- fills
    void zero();
    void ones();
    void fill(float v);

    // ---- views
    Tensor transpose(int dim0, int dim1) const;   // deep copy + stride swap, as the reference
    Tensor t() const;
    Tensor contiguous() const;

    // ---- operators (dispatched)
    Tensor operator+(const Tensor& other) const;
    Tensor operator-(const Tensor& other) const;
    Tensor operator*(const Tensor& other) const;
    Tensor operator/(const Tensor& other) const;
    Tensor operator-() const;
    Tensor matmul(const Tensor& other) const;
    // Not in the reference: `(x.matmul(weight) + bias)` and, with relu, `.relu()` of it
    // (the layer of mnist/mnist.cpp:39-41) as ONE operator: one launch and one tape entry on the
    // device, with the values and gradients of the three-operator form bit for bit.  On the host it
    // is the three operators.
    Tensor linear(const Tensor& weight, const Tensor& bias, bool relu = false) const;
    // Not in the reference: `x.linear(weight, bias).cross_entropy(labels)` with class-index labels
    // (mnist/mnist.cpp:41 and :67-73; CrossEntropy_BASIC_kernel.cpp:88-120) as ONE operator.  For a head
    // of at most 16 classes over at most 256 hidden units the device forms the logits, the loss and -
    // under a tape - the gradients of x, weight and bias in one pass over x; backward() hands them
    // out when the loss is its root (any other upstream gradient rescales the kept gradient of the
    // logits and takes the usual products).  Values agree with the two-operator form within the
    // MatMul bound (the products are added in another order).  It is one node of the tape: a tape that
    // is walked twice without being cleared adds one contribution per pass to x, weight and bias,
    // where the two-operator form's logits node would accumulate too.  Any other shape, a host tensor or
    // one-hot targets: the two operators.  logits (optional) receives x.linear(weight, bias).
    Tensor linear_cross_entropy(const Tensor& weight, const Tensor& bias, const Tensor& labels, Tensor* logits = nullptr) const;
    Tensor dot(const Tensor& other) const;
    Tensor relu() const;
    Tensor sigmoid() const;
    Tensor tanh() const;
    Tensor sin() const;
    Tensor cos() const;
    Tensor mse_loss(const Tensor& target) const;
    Tensor mae_loss(const Tensor& target) const;
    Tensor cross_entropy(const Tensor& target) const;
    // ---- host-inline in the reference, device kernels here
    Tensor operator+(float scalar) const;
    Tensor operator*(float scalar) const;
    Tensor operator/(float scalar) const;
    // elementwise comparisons, DType::kBool results (src/Tensor.cpp:985-1309); not taped
    Tensor operator>(float scalar) const;
    Tensor operator<(float scalar) const;
    Tensor operator==(float scalar) const;
    Tensor operator>=(float scalar) const;
    Tensor operator<=(float scalar) const;
    Tensor operator!=(float scalar) const;
    Tensor operator>(const Tensor& other) const;
    Tensor operator<(const Tensor& other) const;
    Tensor operator==(const Tensor& other) const;
    Tensor operator>=(const Tensor& other) const;
    Tensor operator<=(const Tensor& other) const;
    Tensor operator!=(const Tensor& other) const;   // declared by the reference (Tensor.h), defined here
    std::vector<unsigned char> to_bytes() const;    // the elements' bytes on the host, any dtype (contiguous tensors)
    Tensor sum() const;
    Tensor softmax(int dim = -1) const;
    // ---- declared by the reference (include/Tensor.h:719, :824-1072, :1117) and never defined there;
    // defined here for kAMD float tensors, each taped with its gradient.  Semantics: the C++ library
    // call the name stands for; reductions over `dims` (negative counts from the end; none = all)
    // drop the reduced dimensions unless keepdim; max / min return values only and pass the gradient
    // to the first extreme element; var / std divide by count - 1 (the sample statistics that the
    // API this class imitates returns by default) - var_of / std_of take the correction explicitly;
    // several dimensions must be adjacent for var / std.
    Tensor operator-(float scalar) const;
    Tensor abs() const;
    Tensor exp() const;
    Tensor log() const;
    Tensor sqrt() const;
    Tensor square() const;
    Tensor tan() const;
    Tensor leaky_relu(float negative_slope = 0.01f) const;
    Tensor log_softmax(int dim = -1) const;
    Tensor sum(const std::vector<int>& dims, bool keepdim = false) const;
    Tensor sum(int dim, bool keepdim = false) const;
    Tensor mean(const std::vector<int>& dims, bool keepdim = false) const;
    Tensor mean(int dim, bool keepdim = false) const;
    Tensor mean() const;
    Tensor max(const std::vector<int>& dims, bool keepdim = false) const;
    Tensor max(int dim, bool keepdim = false) const;
    Tensor max() const;
    Tensor min(const std::vector<int>& dims, bool keepdim = false) const;
    Tensor min(int dim, bool keepdim = false) const;
    Tensor min() const;
    Tensor std(const std::vector<int>& dims, bool keepdim = false) const;
    Tensor std(int dim, bool keepdim = false) const;
    Tensor std() const;
    Tensor var(const std::vector<int>& dims, bool keepdim = false) const;
    Tensor var(int dim, bool keepdim = false) const;
    Tensor var() const;
    Tensor var_of(const std::vector<int>& dims, bool keepdim, int ddof) const;
    Tensor std_of(const std::vector<int>& dims, bool keepdim, int ddof) const;
    Tensor matmul_unified(const Tensor& other) const;    // the reference's "unified" product (:1117): matmul

    // ---- autograd
    void backward() const;
    void backward(const Tensor& grad_output) const;
};

void backward(Tensor& root);
void backward(Tensor& root, Tensor grad_output);
Tensor grad(const Tensor& t);
Tensor matMul(const Tensor& a, const Tensor& b);

#include "AutoDiff.h"
#endif
