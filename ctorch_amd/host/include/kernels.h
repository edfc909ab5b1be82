// Kernel ABI of the scheduler: the reference's two function-pointer types
// (src/kernels/kernels.h:23,31) and, following its naming rule <Op>_<PLATFORM>_kernel
// (CONTRIBUTING.md:54-55), the AMD column: one shim per registered operator that unpacks the
// Tensors, allocates the result on the inputs' device and calls the extern "C" launch layer
// (include/ctorch_amd.h).  Same argument meaning, result shapes and error behaviour as the
// CPU-BASIC kernels they stand beside.
#ifndef CTORCH_AMD_HOST_KERNELS_H
#define CTORCH_AMD_HOST_KERNELS_H
#include "Tensor.h"

typedef Tensor (*BinaryKernelFunc)(const Tensor& a, const Tensor& b);
typedef Tensor (*UnaryKernelFunc)(const Tensor& a);

Tensor Add_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor Sub_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor Mul_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor Div_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor MatMul_AMD_kernel(const Tensor& a, const Tensor& b);
// x.matmul(w) + bias (row vector), then ReLU when asked, in one launch; equals the separate kernels bit for bit
Tensor Linear_AMD_kernel(const Tensor& x, const Tensor& w, const Tensor& bias, bool relu);
// (a . b) * [y > 0] in the product's launch: what MatMul's backward branch followed by the ReLU branch
// of the layer that produced y compute (src/AutoDiff.cpp:1692-1704, :1320-1371)
Tensor MatMulReluMask_AMD_kernel(const Tensor& a, const Tensor& b, const Tensor& y);
// a . b, and into `sums` (a new 1-D tensor) the column sums of the contiguous b, with the bits of
// MatMul_AMD_kernel and of the column sum: a layer's weight gradient x^T . dz and its bias gradient
// from one call, in one launch when the layer is small (src/AutoDiff.cpp:1692-1704, :690-757)
Tensor MatMulColSum_AMD_kernel(const Tensor& a, const Tensor& b, Tensor& sums);
Tensor Dot_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor MSE_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor MAE_AMD_kernel(const Tensor& a, const Tensor& b);
Tensor CrossEntropy_AMD_kernel(const Tensor& a, const Tensor& b);

Tensor Neg_AMD_kernel(const Tensor& a);
Tensor ReLU_AMD_kernel(const Tensor& a);
Tensor Cos_AMD_kernel(const Tensor& a);
Tensor Sin_AMD_kernel(const Tensor& a);
Tensor Tanh_AMD_kernel(const Tensor& a);
Tensor Sigmoid_AMD_kernel(const Tensor& a);
Tensor Softmax_AMD_kernel(const Tensor& a);
// leaky ReLU with the default slope of Tensor::leaky_relu (0.01): the kernel that the reference
// declares (src/kernels/kernels.h:201) and registers without a function (Ctorch_Scheduler.h:51-52)
Tensor LReLU_AMD_kernel(const Tensor& a);

namespace ctorch_amd_host {
// Device branches of the arithmetic that the reference runs inline on the host (not behind the
// scheduler): used by the Tensor front-end and the tape.
Tensor scalar_op(const Tensor& a, float s, op which);
// a (cmp) b or, with b == nullptr, a (cmp) s: a bool tensor; cmp is a CTAMD_CMP_* code
Tensor compare_op(int cmp, const Tensor& a, const Tensor* b, float s);                 // a + s, a * s, a / s
Tensor sum_all(const Tensor& a);
// the methods the reference declares without defining them; `which` is op::Abs, Exp, Log, Sqrt,
// Square, Tan or LReLU (param = slope)
Tensor unary_declared(op which, const Tensor& a, float param = 0.0f);
// their gradients; v is the operand (Abs, Log, Square, LReLU) or the result (Exp, Sqrt, Tan)
Tensor unary_declared_backward(op which, const Tensor& v, const Tensor& g, float param = 0.0f);
// sum / mean / max / min / var / std (kind: CTAMD_RED_*) of `a` read as [outer, len, inner] over its
// middle axis; the result has `result_shape`.  index (max / min) and mean (var / std) receive what
// the gradient needs when they are not null.
Tensor reduce_axis(int kind, const Tensor& a, size_t outer, size_t len, size_t inner, int ddof,
                   const std::vector<size_t>& result_shape, Tensor* index, Tensor* mean);
Tensor reduce_axis_backward(int kind, const Tensor& x, const Tensor& y, const Tensor& index, const Tensor& mean, const Tensor& g,
                            size_t outer, size_t len, size_t inner, int ddof);
Tensor log_softmax_dim(const Tensor& a, int dim);                       // dim already normalised
Tensor log_softmax_backward(const Tensor& y, const Tensor& g, int dim);
// gradient shape adjustment beyond the row-vector cases: the modulo fold of shapes that do not
// broadcast, and the sum over / repetition along broadcast dimensions (shapes padded to one rank)
Tensor fold_mod(const Tensor& g, const std::vector<size_t>& target_shape);
Tensor broadcast_reduce(const Tensor& g, const std::vector<size_t>& g_shape, const std::vector<size_t>& t_shape,
                        const std::vector<size_t>& result_shape);
// the first `count` elements of g as a tensor of `shape` (a copy)
Tensor leading_elements(const Tensor& g, const std::vector<size_t>& shape);
// Class-index cross entropy under a tape whose logits need a gradient computes loss and gradient in
// one pass over the logits and keeps the gradient for backward() (default on; off: a forward pass
// that leaves row statistics, and a streaming backward pass).
void set_ce_one_pass(bool on);
// The reference range-checks class indices before it computes and returns an empty Tensor for a bad
// one (CrossEntropy_BASIC_kernel.cpp:96-100); on the device that answer costs a wait for the kernel in
// the middle of a training step.  With the deferred check the loss comes back at once and is NaN for a
// bad index (what a recorded step does anyway).  Off by default.
void set_ce_deferred_label_check(bool on);
bool ce_deferred_label_check();
// A condition that a kernel reports through four bytes on the device and that has to become an
// exception: registered while a backward pass queues its launches, read when the pass has queued
// them all (AutoDiff::backward calls run_deferred_checks before it returns).
void defer_status_check(const Tensor& status, const std::string& message);
void run_deferred_checks();
void drop_deferred_checks();
void set_ce_kept_bytes(size_t cap);   // most bytes of one-pass CrossEntropy gradients kept for a backward() (default 4 GiB)
size_t ce_kept_bytes();
bool ce_one_pass();
// tensors that are not fp32 (the typed arms of src/Tensor.cpp:197-243, :390-448)
void fill_typed(void* device_ptr, DType dtype, double v, size_t n);    // zero() / ones() of any dtype, device memory
Tensor cast_from_float(const Tensor& a, DType to);                    // Tensor::to(DType)
Tensor softmax_dim(const Tensor& a, int dim);                         // dim already normalised
Tensor filled(const std::vector<size_t>& shape, float v, DeviceType device);
void fill_scalar(Tensor& t, float v);                                  // every element of a device tensor = v
Tensor filled_from(const std::vector<size_t>& shape, const Tensor& scalar0d);
void accumulate(Tensor& grad, const Tensor& val);                     // grad += val
Tensor zero_plus(const Tensor& val, const std::vector<size_t>& shape); // a fresh tensor: 0 + val
Tensor sum_of(const Tensor& a, const Tensor& b);                       // a fresh tensor: a + b, a's shape
Tensor column_sum(const Tensor& g);                                   // [rows, cols] -> [cols]
Tensor first_row(const Tensor& g);                                    // [rows, cols] -> [cols], row 0
bool any_abs_lt_eps(const Tensor& b);
void copy_into(Tensor& dst, const Tensor& src);                        // device-to-device, same element count
// the MNIST demo's host loops as device launches
Tensor onehot(const Tensor& labels, size_t classes);                   // mnist/mnist.cpp:72-78
void sgd_step(Tensor& param, const Tensor& grad, float lr);            // mnist/mnist.cpp:86-92, in place
// the same update for several parameters in one launch; grads as AutoDiff::stored_grad returns them
// (an empty gradient leaves its parameter alone), "0 +" applied in the kernel
void sgd_step_all(const std::vector<Tensor*>& params, const std::vector<Tensor>& grads, float lr);
size_t count_correct(const Tensor& pred, const Tensor& labels);        // mnist/mnist.cpp:134-156 (reads back)
Tensor unit_from_bytes(const unsigned char* host_bytes, size_t rows, size_t cols);  // mnist_loader.cpp:33-41
Tensor relu_backward(const Tensor& x, const Tensor& g);
Tensor sigmoid_backward(const Tensor& x, const Tensor& g);
Tensor tanh_backward(const Tensor& x, const Tensor& g);
Tensor sin_backward(const Tensor& x, const Tensor& g);
Tensor cos_backward(const Tensor& x, const Tensor& g);
Tensor softmax_backward(const Tensor& y, const Tensor& g, int dim);
Tensor mse_backward(const Tensor& p, const Tensor& t, const Tensor& g0d);
Tensor mae_backward(const Tensor& p, const Tensor& t, const Tensor& g0d);
// acc + the gradient of ReLU / Sigmoid / Tanh / Sin / Cos at x, in the pass that forms it
Tensor unary_backward_plus(op which, const Tensor& x, const Tensor& g, const Tensor& acc);
// acc + g / b (the quotient rounded first), one pass; b of g's shape or a row vector under it
Tensor div_plus(const Tensor& g, const Tensor& b, const Tensor& acc);
// acc + a * b (the product rounded first), one pass
Tensor mul_plus(const Tensor& a, const Tensor& b, const Tensor& acc);
// acc + the MSE (mae = false) or MAE gradient, in the pass that forms it
Tensor loss_backward_plus(bool mae, const Tensor& p, const Tensor& t, const Tensor& g0d, const Tensor& acc);
Tensor cross_entropy_backward(const Tensor& x, const Tensor& target, const Tensor& g0d);
// The classifier head in one pass (ctamd_linear_ce_head_f32); whether the shapes fit it, and the call:
// returns the loss (an empty Tensor for a class index out of range, as CrossEntropy_AMD_kernel), fills
// the gradient of the logits for an upstream gradient of 1, of the weights and of the bias, the
// logits when wanted, and dh (times [h > 0] when mask_by_h) when wanted.
bool linear_ce_head_fits(const Tensor& h, const Tensor& w, const Tensor& bias, const Tensor& labels);
Tensor linear_ce_head(const Tensor& h, const Tensor& w, const Tensor& bias, const Tensor& labels, bool mask_by_h, Tensor* logits,
                      Tensor& dz, Tensor* dh, Tensor& gw, Tensor& gb);
Tensor div_backward_b(const Tensor& a, const Tensor& b, const Tensor& g);
// The stream every launch of this front-end goes to (as the C ABI's void*): the null stream unless a
// DeviceGraph is recording or has installed its own.  While a graph records, anything that would
// make the host wait for the device (item(), to_vector(), a transfer, a pool trim) throws.
void* current_stream();
void set_current_stream(void* stream);
bool recording();
void set_recording(bool on);
void init_device();   // ctamd_init(0), once; throws if there is no gfx950 device
}  // namespace ctorch_amd_host
#endif
