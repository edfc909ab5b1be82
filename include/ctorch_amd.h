/* ctorch_amd - C ABI of the MI355X (gfx950) device backend for CTorch's operator set.
 *
 * One entry point per kernel the reference registers in Ctorch_Scheduler
 * (include/Ctorch_Scheduler.h:30-53) or runs inline in its Tensor front-end / tape
 * (src/Tensor.cpp, src/AutoDiff.cpp).  Each declaration cites the reference code it replaces
 * (paths relative to the reference root).
 *
 * Conventions
 *  - Every pointer is DEVICE memory (HBM) unless its name ends in _host.  All data is fp32,
 *    row-major, contiguous unless strides are passed.  Counts are in elements.
 *  - Launchers never allocate, free or synchronise: they enqueue on `stream` (a hipStream_t passed
 *    as void*, NULL = the default stream) and return.  Results are ready after ctamd_sync(stream).
 *  - Reductions, losses, column softmax / sums and matrix products whose tiles are cut along K use
 *    a per-device scratch buffer that ctamd_init() allocates once.  All streams of a device share
 *    it, and the library puts them in order: a call on another stream than the previous such call
 *    makes its stream wait (on the device) for the previous stream's scratch-using work, through an
 *    event the library records after that work.  So such calls run one after another across streams,
 *    never at once.  While a graph is being recorded the scratch belongs to the recording (other
 *    streams get CTAMD_EINVAL); replays take their turn through ctamd_graph_launch.  Work recorded
 *    into a graph by other means than ctamd_graph_begin / _end is not tracked at replay.
 *  - Math mode (ctamd_set_math_mode): CTAMD_MATH_FAST, the default, evaluates the exponentials of
 *    softmax / log-softmax / cross entropy and the sigmoid, sin, cos of fused expressions in single
 *    precision within 2 ulp of the reference's libm loops (a fused tanh keeps the reference's bits:
 *    its quotient of exponentials amplifies any other rounding); CTAMD_MATH_EXACT returns the bits of
 *    those loops everywhere.  The one-operator kernels return glibc's floats in both modes.
 *  - Return value: 0 on success, a negative CTAMD_E* code otherwise; ctamd_last_error() gives
 *    the text.  No C++ exception crosses this boundary.  The C++ shim above maps codes to the
 *    reference's two error conventions (Ctorch_Error::log / throwException,
 *    include/Ctorch_Error.h:353-405, :510-515).
 *  - n == 0 (and rows == 0 or cols == 0) is a successful no-op.
 */
#ifndef CTORCH_AMD_H
#define CTORCH_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CTAMD_OK 0
#define CTAMD_EINVAL (-1)   /* bad argument: null pointer, negative size, bad op code, shape mismatch */
#define CTAMD_EHIP (-2)     /* the HIP runtime reported an error (launch, copy, allocation) */
#define CTAMD_ENOMEM (-3)   /* device allocation failed */
#define CTAMD_ENODEV (-4)   /* no gfx950 device visible */
#define CTAMD_ERANGE (-5)   /* a size exceeds what the entry point supports */

/* ------------------------------------------------------------------------------- runtime */

/* Selects device `device`, checks it is a gfx950 part and allocates the reduction scratch.
 * Idempotent.  Replaces the device gate Ctorch_Scheduler::isDeviceAvailable
 * (include/Ctorch_Scheduler.h:67-75). */
int ctamd_init(int device);
int ctamd_device_count(void);
const char* ctamd_last_error(void);
const char* ctamd_version(void);

/* How softmax, log_softmax's gradient, the cross-entropy gradients and the fused expressions evaluate
 * exp / sin / cos (process-wide; takes effect for later launches).  The reference calls glibc's expf,
 * sinf, cosf (src/Tensor.cpp:1682,1722; src/AutoDiff.cpp:1558,1564; CrossEntropy_BASIC_kernel.cpp:56).
 *   CTAMD_MATH_FAST  (default) single precision, within 2 ulp of those calls, and e * (1 / sum) for
 *                    the softmax quotient: the kernels run at memory speed
 *   CTAMD_MATH_EXACT the double-precision routines that return glibc 2.35's floats bit for bit and
 *                    the exactly rounded quotient e / sum, as the reference computes it; 1.2 - 2x slower
 * The one-operator kernels (ctamd_sin_f32, ctamd_exp_f32, ...) always return glibc's floats. */
#define CTAMD_MATH_FAST 0
#define CTAMD_MATH_EXACT 1
int ctamd_set_math_mode(int mode);
int ctamd_math_mode(void);

/* Storage: device allocation and explicit transfers; replaces `new char[]` / memcpy in
 * Storage (include/Storage.h:77, :175-181). */
int ctamd_malloc(void** ptr, size_t bytes);
int ctamd_free(void* ptr);
int ctamd_memcpy_h2d(void* dst, const void* src_host, size_t bytes, void* stream);
int ctamd_memcpy_d2h(void* dst_host, const void* src, size_t bytes, void* stream);
int ctamd_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int ctamd_sync(void* stream);
/* Tensor::item<T>() (include/Tensor.h:642-660) and the other reads of a few bytes that a training loop
 * makes every step (a loss, a Dot, a status word): `bytes` <= CTAMD_READ_SMALL_MAX from device memory into
 * host memory once the work queued on `stream` is done.  The copy goes into a page-locked buffer the
 * library keeps per host thread, so it is queued behind that work at once and the host waits a single
 * time; a copy into pageable memory makes the host wait for the stream, copy, and wait again. */
#define CTAMD_READ_SMALL_MAX 256
int ctamd_read_small(void* dst_host, const void* src, size_t bytes, void* stream);

/* Streams and recorded launch sequences, with no counterpart in the reference (which is
 * synchronous): a caller whose step is a fixed sequence of small launches (a training step at a
 * small batch costs ~3 us of launch overhead per operator) records it once into a HIP graph and
 * replays it with one launch.  ctamd_graph_begin(stream) puts a stream created by
 * ctamd_stream_create into recording mode: every launcher called with that stream until
 * ctamd_graph_end is recorded, not executed.  No entry point records a memset node (flags and
 * counters are cleared by kernels), so every launcher is safe to record; ctamd_sync, the h2d/d2h
 * copies and ctamd_malloc/free are not stream work and must not be called on a recording stream.
 * The recorded sequence holds the device pointers it was recorded with. */
int ctamd_stream_create(void** stream);
int ctamd_stream_destroy(void* stream);
int ctamd_graph_begin(void* stream);
int ctamd_graph_end(void* stream, void** graph);
int ctamd_graph_launch(void* graph, void* stream);
int ctamd_graph_destroy(void* graph);

/* Work counters, a measurement aid with no counterpart in the reference.  Every operator entry
 * point below adds its algorithmic HBM bytes and flops (what the operator must move and compute:
 * e.g. 12 bytes per element for r = a + b, 2*m*n*k flops for MatMul), and
 * max(bytes / 8 TB/s, flops / 157.3 TFLOP/s), the time that work takes at the MI355X peaks, to
 * per-process totals.  roofline_seconds / measured seconds is the roofline fraction of whatever
 * sequence of operators ran between a reset and a read.  Any pointer may be NULL. */
void ctamd_counters_reset(void);
void ctamd_counters_read(double* bytes, double* flops, double* roofline_seconds, uint64_t* launches);

/* -------------------------------------------------------- elementwise binary (bit-exact) */
/* r[i] = a[i] (op) b[i].  Add_BASIC_kernel.cpp:64-69, Sub_BASIC_kernel.cpp:58-60,
 * Mul_BASIC_kernel.cpp:59-61, Div_BASIC_kernel.cpp:37-45 (IEEE quotient, also for b == 0). */
int ctamd_add_f32(const float* a, const float* b, float* r, size_t n, void* stream);
int ctamd_sub_f32(const float* a, const float* b, float* r, size_t n, void* stream);
int ctamd_mul_f32(const float* a, const float* b, float* r, size_t n, void* stream);
int ctamd_div_f32(const float* a, const float* b, float* r, size_t n, void* stream);

/* r[i,j] = a[i,j] (op) b[j], a [rows, cols], b [cols].  Add_BASIC_kernel.cpp:27-29, :54-63.
 * The reference has this form for Add only; Sub/Mul/Div follow the same convention here
 * (the reference throws for Sub/Mul and reads out of bounds for Div:
 * Sub_BASIC_kernel.cpp:35-43, Tensor.cpp:362-365, Div_BASIC_kernel.cpp:18-20). */
int ctamd_add_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* stream);
int ctamd_sub_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* stream);
int ctamd_mul_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* stream);
int ctamd_div_rowbcast_f32(const float* a, const float* b, float* r, size_t rows, size_t cols, void* stream);

/* r[i] = a[i] (op) b[0] with b a one-element DEVICE tensor.  Add_BASIC_kernel.cpp:48-53; for
 * Sub/Mul the 0-D broadcast branch (Sub_BASIC_kernel.cpp:28-32, Mul_BASIC_kernel.cpp:27-34). */
int ctamd_add_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* stream);
int ctamd_sub_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* stream);
int ctamd_mul_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* stream);
int ctamd_div_bscalar_f32(const float* a, const float* b1, float* r, size_t n, void* stream);
/* r[i] = a1[0] - b[i]: a 0-D left operand (Sub_BASIC_kernel.cpp:25-27), used by the tape for
 * 1 - sigmoid(x) and 1 - tanh(x)^2 (src/AutoDiff.cpp:1379, :1393). */
int ctamd_rsub_ascalar_f32(const float* a1, const float* b, float* r, size_t n, void* stream);

/* r[i] = a[i] (op) s with s a HOST float.  Tensor::operator+(float) src/Tensor.cpp:855-910,
 * operator*(float) :751-806, operator/(float) :913-973. */
int ctamd_add_scalar_f32(const float* a, float s, float* r, size_t n, void* stream);
int ctamd_mul_scalar_f32(const float* a, float s, float* r, size_t n, void* stream);
int ctamd_div_scalar_f32(const float* a, float s, float* r, size_t n, void* stream);

/* ---------------------------------------------------------------------- elementwise unary */
/* Neg_BASIC_kernel.cpp:26-28 (sign-bit flip); ReLU_BASIC_kernel.cpp:23-25 (x > 0 ? x : +0, so
 * -0 and NaN give +0): bit-exact. */
int ctamd_neg_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_relu_f32(const float* a, float* r, size_t n, void* stream);
/* Sin_BASIC_kernel.cpp:24-26, Cos_BASIC_kernel.cpp:23-25 (glibc sinf / cosf);
 * Tanh_BASIC_kernel.cpp:24-28 ((e^x - e^-x) / (e^x + e^-x) in fp32);
 * Sigmoid_BASIC_kernel.cpp:24-26 (1 / (1 + e^-x)).  The device evaluates the same formulas on
 * exp/sin/cos that return glibc 2.35's floats (see ctorch_amd/csrc/devmath.h). */
int ctamd_sin_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_cos_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_tanh_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_sigmoid_f32(const float* a, float* r, size_t n, void* stream);

/* Operators that the reference declares on Tensor and never defines (include/Tensor.h:719 operator-
 * (float), :954-972 abs / exp / log / sqrt, :978 square, :996 tan, :1052 leaky_relu; the kernel
 * LReLU_BASIC_kernel is declared at src/kernels/kernels.h:201 and registered without a function at
 * include/Ctorch_Scheduler.h:51-52).  With no reference arithmetic to follow, each is the C++ library
 * call its name stands for, on floats: a - s; std::fabs; expf, logf (glibc 2.35's floats, bit for
 * bit); IEEE sqrt; a * a; tanf (within 1 ulp of glibc's); x > 0 ? x : x * slope. */
int ctamd_sub_scalar_f32(const float* a, float s, float* r, size_t n, void* stream);
int ctamd_abs_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_exp_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_log_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_sqrt_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_square_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_tan_f32(const float* a, float* r, size_t n, void* stream);
int ctamd_leaky_relu_f32(const float* a, float slope, float* r, size_t n, void* stream);

/* ------------------------------------------------------------------------------- reductions */
/* out[0] = sum of a.  Tensor::sum() src/Tensor.cpp:638-666. */
int ctamd_sum_f32(const float* a, float* out, size_t n, void* stream);
/* out[0] = sum a[i]*b[i].  Dot_BASIC_kernel.cpp:38-41. */
int ctamd_dot_f32(const float* a, const float* b, float* out, size_t n, void* stream);
/* out[0] = sum (a-b)^2 / n and sum |a-b| / n.  MSE_BASIC_kernel.cpp:35-43, MAE_BASIC_kernel.cpp:35-43. */
int ctamd_mse_f32(const float* a, const float* b, float* out, size_t n, void* stream);
int ctamd_mae_f32(const float* a, const float* b, float* out, size_t n, void* stream);
/* ctamd_dot_f32 for callers that cannot allocate device memory or depend on memory the library
 * allocated: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference.  The per-block partial sums live in a 16 KiB array that is
 * part of the library's device image (one copy per GPU, held until the process ends) instead of the
 * scratch buffer ctamd_init() allocates; the call allocates and frees nothing.  Same kernels, same
 * grid and therefore the same bits as ctamd_dot_f32.  n above CTAMD_DOT_STATIC_MAX_N (2^31 - 1,
 * this entry point's stated maximum) is refused with CTAMD_ERANGE and nothing is launched.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two
 * streams, two host threads) race; calls on one stream are ordered.  Nothing needs clearing between
 * calls - the fold launch reads only the partials its own first launch wrote. */
#define CTAMD_DOT_STATIC_MAX_N ((size_t)2147483647)
int ctamd_dot_static_f32(const float* a, const float* b, float* out, size_t n, void* stream);
/* sum / mean / max / min / var / std along one axis: x is read as [outer, len, inner] (row-major) and
 * out[o, i] is the reduction of x[o, :, i].  outer = inner = 1 reduces a whole tensor, inner = 1 the
 * rows of a matrix, outer = 1 its columns.  These are Tensor::sum(dim) / mean / max / min / var / std,
 * which the reference declares and never defines (include/Tensor.h:824-948); the arithmetic fixed
 * here: fp32 terms added in a tree (sum), float(sum) / float(len) (mean), the extreme value and, in
 * index (may be NULL), the position of its FIRST occurrence along the axis (NaN wins only from position 0, as a loop
 * `if (v > m) m = v` started at element 0 behaves), var = sum((x - mean)^2) / (len - ddof) formed in
 * double, std its square root; mean_out (var / std only, may be NULL) receives the mean that the
 * gradient needs.  len <= 2^31 - 1.  Uses the per-device scratch. */
enum { CTAMD_RED_SUM = 0, CTAMD_RED_MEAN = 1, CTAMD_RED_MAX = 2, CTAMD_RED_MIN = 3, CTAMD_RED_VAR = 4, CTAMD_RED_STD = 5 };
int ctamd_reduce_dim_f32(int kind, const float* x, float* out, int32_t* index, float* mean_out, size_t outer, size_t len,
                         size_t inner, int ddof, void* stream);
/* Their gradients, dx of x's shape from g of out's shape: sum g; mean g / float(len); max / min g at
 * index[o, i] and +0 elsewhere; var ((x - mean) * 2 / float(len - ddof)) * g; std
 * ((x - mean) / (float(len - ddof) * y)) * g, each step rounded to fp32 in that order.  x and mean are
 * read by var / std only, y by std only, index by max / min only (others may be NULL). */
int ctamd_reduce_dim_backward_f32(int kind, const float* x, const float* y, const int32_t* index, const float* mean,
                                  const float* g, float* dx, size_t outer, size_t len, size_t inner, int ddof, void* stream);
/* out[i] = g[i] + g[i + out_count] + g[i + 2 * out_count] + ... added in that order from 0: what the
 * reference's check_and_adjust_grad_shape does with a gradient whose shape does not broadcast to the
 * operand's (src/AutoDiff.cpp:968-1046). */
int ctamd_fold_mod_f32(const float* g, float* out, size_t g_count, size_t out_count, void* stream);
/* The gradient of an operand that was broadcast to the gradient's shape, for any shapes of up to 8
 * dimensions: g_shape and t_shape (HOST arrays of `rank` extents, the operand's shape padded with
 * leading 1s) agree per dimension, or the operand's extent is 1 (out sums g over that dimension, in
 * double), or the gradient's is 1 (its value is repeated).  The mathematically complete form of
 * check_and_adjust_grad_shape's broadcast branch (src/AutoDiff.cpp:690-890, which takes one slice
 * instead of the sum); ctamd_colsum_f32 is its [rows, cols] -> [cols] case at memory speed. */
int ctamd_broadcast_reduce_f32(const float* g, const size_t* g_shape, const size_t* t_shape, int rank, float* out, void* stream);
/* out[j] = sum_i g[i,j], g [rows, cols]: the complete gradient of a row-broadcast operand
 * (the reference's check_and_adjust_grad_shape, src/AutoDiff.cpp:690-757, returns row 0 instead;
 * that behaviour is a ctamd_memcpy_d2d of the first row followed by ctamd_accumulate_f32). */
int ctamd_colsum_f32(const float* g, float* out, size_t rows, size_t cols, void* stream);
/* flag[0] = 1 if any |b[i]| < FLT_EPSILON else 0: the divisor scan of Div's backward
 * (src/AutoDiff.cpp:1267-1284). */
int ctamd_any_abs_lt_eps_f32(const float* b, int32_t* flag, size_t n, void* stream);

/* ---------------------------------------------------------------- softmax and cross entropy */
/* Row softmax y[i,:] = softmax(x[i,:]) (dim 1 / 1-D with rows = 1) and column softmax (dim 0).
 * Tensor::softmax src/Tensor.cpp:1713-1727, :1728-1744; Softmax_BASIC_kernel.cpp:72-93.
 * exp(x - max) is bit-identical to the reference's, the row sum is a tree sum, and the
 * normalisation is a true division as in the reference. */
int ctamd_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols, void* stream);
int ctamd_softmax_cols_f32(const float* x, float* y, size_t rows, size_t cols, void* stream);
/* Tensor::log_softmax(dim), declared by the reference and never defined (include/Tensor.h:1072):
 * y = (x - max) - log(sum_j exp(x_j - max)) per row (dim 1 / 1-D) or per column (dim 0), in the style
 * of Tensor::softmax (src/Tensor.cpp:1713-1744): the maximum subtracted first, expf terms of glibc's
 * bits summed in a tree, glibc's logf of the sum; rows of 2048 columns or more and matrices of 128
 * rows or more (columns) form the sum from the hardware exponential (~1e-7 relative).  Gradient:
 * dx = g - exp(y) * sum_j g_j. */
int ctamd_log_softmax_rows_f32(const float* x, float* y, size_t rows, size_t cols, void* stream);
int ctamd_log_softmax_cols_f32(const float* x, float* y, size_t rows, size_t cols, void* stream);
int ctamd_log_softmax_backward_rows_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream);
int ctamd_log_softmax_backward_cols_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols, void* stream);
/* out[0] = SUM over rows of -sum_j t[i,j] * log(max(softmax(x)[i,j], 1e-10)).
 * CrossEntropy_BASIC_kernel.cpp:41-66 (2-D one-hot or soft targets), :67-82 (1-D: rows = 1). */
int ctamd_cross_entropy_onehot_f32(const float* x, const float* t, float* out, size_t rows, size_t cols,
                                   void* stream);
/* Class-index targets held as floats, truncated toward zero.  CrossEntropy_BASIC_kernel.cpp:88-120.
 * status[0] is set to 1 when an index is out of range (the reference then returns an empty
 * Tensor, :96-100) and out[0] is then NaN; status may be NULL. */
int ctamd_cross_entropy_index_f32(const float* x, const float* idx, float* out, int32_t* status, size_t rows,
                                  size_t cols, void* stream);
/* The same, also leaving each row's (max, sum_j exp(x_j - max)) in stats[2*row], stats[2*row+1]
 * (stats may be NULL), and the backward pass that uses them instead of recomputing the row
 * reductions: dx = (exp(x - max) / sum - onehot(idx)) * g1[0], one streaming pass.  The sum of a
 * long row (2048 columns or more) comes from the forward pass's fast exponential, ~1e-7 relative
 * from the sum of the rounded terms. */
int ctamd_cross_entropy_index_stats_f32(const float* x, const float* idx, float* out, int32_t* status, float* stats,
                                        size_t rows, size_t cols, void* stream);
int ctamd_cross_entropy_backward_index_stats_f32(const float* x, const float* idx, const float* stats, const float* g1,
                                                 float* dx, size_t rows, size_t cols, void* stream);
/* Loss and gradient of the logits from ONE visit of each row: out[0] and status[0] as
 * ctamd_cross_entropy_index_f32, and dx = exp(x - max) / sum - onehot(idx), the gradient of
 * src/AutoDiff.cpp:1517-1601 for an upstream gradient of 1 (x * 1.0f is x), which is what a loss that
 * is the root of backward() receives.  The row stays in registers between the two uses: 8 bytes per
 * element instead of the 12 of a forward pass and a backward pass.  Rows of at most 32768 columns
 * (8192 when the row length is no multiple of four or a tensor is not 16-byte aligned); CTAMD_ERANGE
 * beyond, with nothing launched.  Rows of 2048 columns or more use the hardware exponential and a
 * multiplication by 1 / sum (<= 2e-7 from the exact form, as ctamd_cross_entropy_backward_index_stats_f32);
 * shorter rows are bit-equal to ctamd_cross_entropy_backward_index_f32 with g1 = 1.  The reference
 * computes the two in separate passes (CrossEntropy_BASIC_kernel.cpp:88-120,
 * then the tape). */
int ctamd_cross_entropy_index_fused_f32(const float* x, const float* idx, float* out, int32_t* status, float* dx,
                                        size_t rows, size_t cols, void* stream);

/* The classifier head of a small network - the last layer, its cross entropy and every gradient that
 * flows out of them - in one pass over the hidden activations h [batch, hidden]:
 *   z = h . w + bias (mnist/mnist.cpp:41), out[0] / status[0] as ctamd_cross_entropy_index_f32 (the SUM
 *   over rows of -log(max(softmax(z)[label], 1e-10)), CrossEntropy_BASIC_kernel.cpp:88-120),
 *   dz = softmax(z) - onehot(label) (src/AutoDiff.cpp:1517-1601 for an upstream gradient of 1),
 *   dh = dz . w^T (src/AutoDiff.cpp:1684-1704), times [h > 0] when mask_by_h is set (the ReLU branch
 *   :1320-1371 of the layer that produced h), gw = h^T . dz (:1766-1810), gb = the column sums of dz.
 * z and dh may be null.  2 to 16 classes, hidden a multiple of four up to 256 (ctamd_linear_ce_head_fits
 * tells), h and dh 16-byte aligned; CTAMD_ERANGE otherwise with nothing launched.  fp32 fused
 * multiply-adds in a fixed order (deterministic), so products differ from ctamd_matmul_f32's in the last
 * bits: equal to the five separate launches within the MatMul bound.  Uses the per-device scratch.
 * The reference runs the five steps as separate kernels and tape branches. */
int ctamd_linear_ce_head_fits(size_t hidden, size_t classes);
int ctamd_linear_ce_head_f32(const float* h, const float* w, const float* bias, const float* labels, float* out, int32_t* status,
                             float* z, float* dz, float* dh, int mask_by_h, float* gw, float* gb, size_t batch, size_t hidden,
                             size_t classes, void* stream);

/* -------------------------------------------------------------------------------- matmul */
/* C[i,j] = sum_l A[i*as0 + l*as1] * B[l*bs0 + j*bs1]; C is [m, n] row-major contiguous; strides
 * are in elements and may describe a transposed view.  MatMul_BASIC_kernel.cpp:42-54.  The
 * reference's backward calls the same kernel with t() views: dA = g.matmul(B.t()),
 * dB = A.t().matmul(g) (src/AutoDiff.cpp:1692-1704, :1808-1810).  fp32 MFMA with fp32
 * accumulation; every operand layout with a unit stride in one dimension takes the MFMA path
 * (products with at most 16 output columns that are too large for one launch of small MFMA
 * tiles: fp32 FMAs on the vector units, in a fixed order), anything else a generic strided
 * kernel.  Results are deterministic: the same call gives the same bits. */
int ctamd_matmul_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                     float* c, int64_t m, int64_t n, int64_t k, void* stream);

/* One layer of the demo network in one launch: C = A.B, then "+ bias" broadcast over rows (bias
 * [n], may be NULL), then ReLU when relu != 0 -- the sequence matmul, operator+, relu() of
 * mnist/mnist.cpp:39-41 (MatMul_BASIC_kernel.cpp:42-54, Add_BASIC_kernel.cpp:54-63,
 * ReLU_BASIC_kernel.cpp:19-25).  Each step rounds as its own kernel does, so the result equals
 * ctamd_matmul_f32, ctamd_add_rowbcast_f32, ctamd_relu_f32 in sequence bit for bit. */
int ctamd_matmul_bias_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                          const float* bias, int relu, float* c, int64_t m, int64_t n, int64_t k, void* stream);

/* c = a . b as ctamd_matmul_f32 computes it, and sums[j] = sum over k of b[k, j] as
 * ctamd_colsum_f32(b, sums, k, n) computes it - the same bits as the two calls: the weight gradient
 * x^T . dz of a layer and its bias gradient, the column sums of dz (the tape's MatMul branch,
 * src/AutoDiff.cpp:1692-1704, and the reduction of a broadcast operand's gradient, :690-757).  b must
 * lie in contiguous rows (CTAMD_EINVAL otherwise, nothing launched).  When the product is small enough
 * for the one-launch small-product kernel (at most 256 tiles of 32 x 32, k <= 512), the sums are
 * computed by extra blocks of that launch: one kernel on the chain of dependent launches instead of
 * two.  When the product is cut along K on the 64 x 64 tiles (a long k over a few hundred columns: the
 * weight gradient of a small layer at a large batch) and b has at most 512 columns in 16-byte aligned
 * rows, the first stage of the column sum runs as extra blocks of the product's launch and the second as
 * extra blocks of the launch that adds the parts: two launches instead of four.  Every other shape runs
 * the two operators one after the other. */
int ctamd_matmul_colsum_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                            float* c, float* sums, int64_t m, int64_t n, int64_t k, void* stream);

/* The gradient that reaches a ReLU layer's pre-activation, formed by the product that computes it:
 * C = (A.B) * [y > 0], y the [m, n] row-major output of that ReLU.  The reference computes the
 * product in the MatMul branch of backward (g.matmul(B.t()), src/AutoDiff.cpp:1692-1704) and the
 * mask in the ReLU branch of the layer below (grad * [x > 0], :1320-1371; y > 0 exactly where
 * x > 0); here the factor 0 / 1 multiplies the accumulator as it is stored.  Equal to
 * ctamd_matmul_f32 followed by ctamd_relu_backward_f32(y, C, C) bit for bit. */
int ctamd_matmul_relu_mask_f32(const float* a, int64_t as0, int64_t as1, const float* b, int64_t bs0, int64_t bs1,
                               const float* y, float* c, int64_t m, int64_t n, int64_t k, void* stream);

/* -------------------------------------------------------------------------- comparisons */
/* out[i] = (a[i] cmp b[i]) or (a[i] cmp s) as one byte, 0 or 1 - the reference's bool tensors.
 * Tensor::operator>,<,==,>=,<=,!=(float) src/Tensor.cpp:985-1116 and (const Tensor&) :1119-1309;
 * IEEE comparisons (anything against NaN is false, != is true). */
enum { CTAMD_CMP_GT = 0, CTAMD_CMP_LT = 1, CTAMD_CMP_EQ = 2, CTAMD_CMP_GE = 3, CTAMD_CMP_LE = 4, CTAMD_CMP_NE = 5 };
int ctamd_compare_f32(int cmp, const float* a, const float* b, uint8_t* out, size_t n, void* stream);
int ctamd_compare_scalar_f32(int cmp, const float* a, float s, uint8_t* out, size_t n, void* stream);

/* ------------------------------------------------------- tensors that are not fp32 */
/* The reference's arms for double, int32, int64 and bool tensors.  dtype codes are the order of
 * enum DType (include/Ctools.h:163-169).  Tensors start on 16-byte boundaries and are contiguous.
 * Integer arithmetic wraps; fp32 -> integer conversion truncates and gives the most negative
 * integer for NaN and for values out of range, as the reference's x86 build does. */
enum { CTAMD_DT_F32 = 0, CTAMD_DT_F64 = 1, CTAMD_DT_I32 = 2, CTAMD_DT_I64 = 3, CTAMD_DT_BOOL = 4 };
/* out[i] = value converted to dtype (bool: value != 0): Tensor::zero() / ones()
 * src/Tensor.cpp:390-448 and the zero tensors of AutoDiff::get_grad src/AutoDiff.cpp:205-245. */
int ctamd_fill_typed(void* out, int dtype, double value, size_t n, void* stream);
/* out[i] = static_cast<T>(in[i]) for T = double, int32, int64, bool: Tensor::to(DType)
 * src/Tensor.cpp:197-243 (which converts from fp32 only). */
int ctamd_cast_from_f32(const float* in, void* out, int dtype, size_t n, void* stream);
/* out[i] = in[i] op static_cast<T>(scalar) for T = double, int32, int64: the typed arms of
 * Tensor::operator+(float) src/Tensor.cpp:870-890, operator*(float) :766-786, operator/(float)
 * :933-953.  Integer division truncates; CTAMD_EINVAL when the scalar converts to the integer 0
 * (the reference's process stops with SIGFPE there); the most negative integer divided by -1
 * wraps to itself (the reference stops there as well). */
enum { CTAMD_TS_ADD = 0, CTAMD_TS_MUL = 1, CTAMD_TS_DIV = 2 };
int ctamd_scalar_op_typed(const void* in, void* out, int dtype, int op, float scalar, size_t n, void* stream);
/* acc[i] += val[i] for double, int32, int64: the typed arms of the gradient accumulation
 * src/AutoDiff.cpp:1880-1903. */
int ctamd_accumulate_typed(void* acc, const void* val, int dtype, size_t n, void* stream);
/* Softmax of a double tensor along dim 1 (rows; a 1-D tensor is one row) or dim 0 (columns):
 * Tensor::softmax(dim) src/Tensor.cpp:1686-1696, :1747-1783.  exp is the device library's double
 * exponential, not glibc's: results agree with the reference's to a few units in the last place. */
int ctamd_softmax_f64(const double* x, double* y, size_t rows, size_t cols, int dim, void* stream);

/* ------------------------------------------------------------------ fused expressions */
/* A chain of the elementwise operators above evaluated in ONE pass over memory: the front-end
 * compiles an expression such as Y = sigmoid(X / r) - tanh(X) * sin(X) + cos(-X) (and, separately,
 * its tape gradients) into a straight-line program over value slots.  Every operator computes
 * exactly what its one-operator entry point computes, so a program's results equal the
 * operator-by-operator evaluation bit for bit.  No counterpart in the reference, which runs one
 * kernel per operator (src/Tensor.cpp dispatch sites); the operator semantics are those of
 * Add/Sub/Mul/Div/Neg/ReLU/Sigmoid/Tanh/Sin/Cos_BASIC_kernel.cpp, Tensor::operator+,*,/(float)
 * (src/Tensor.cpp:751-973) and the gradient formulas of src/AutoDiff.cpp:1216-1416. */
enum {
    CTAMD_EX_LOAD_FULL = 0, /* slot[dst] = inputs[a][i]            ([rows, cols] tensor)            */
    CTAMD_EX_LOAD_ROW = 1,  /* slot[dst] = inputs[a][i % cols]     (row vector [cols])              */
    CTAMD_EX_ADD = 2,       /* slot[dst] = slot[a] + slot[b]; SUB, MUL, DIV alike                   */
    CTAMD_EX_SUB = 3,
    CTAMD_EX_MUL = 4,
    CTAMD_EX_DIV = 5,
    CTAMD_EX_NEG = 6,       /* slot[dst] = f(slot[a])                                               */
    CTAMD_EX_RELU = 7,
    CTAMD_EX_SIGMOID = 8,
    CTAMD_EX_TANH = 9,
    CTAMD_EX_SIN = 10,
    CTAMD_EX_COS = 11,
    CTAMD_EX_ADDS = 12,     /* slot[dst] = slot[a] + imm; MULS: * imm; DIVS: / imm                  */
    CTAMD_EX_MULS = 13,
    CTAMD_EX_DIVS = 14,
    CTAMD_EX_RSUBS = 15,    /* slot[dst] = imm - slot[a]                                            */
    CTAMD_EX_RELUMUL = 16,  /* slot[dst] = slot[b] * (slot[a] > 0 ? 1 : 0)    (ReLU's gradient)     */
    CTAMD_EX_DIVCHK = 17,   /* status[0] |= 1 if |slot[a]| < FLT_EPSILON anywhere                   */
    CTAMD_EX_STORE = 18,    /* outputs[dst][i] = slot[a]                                            */
    CTAMD_EX_STORE_ZP = 19  /* outputs[dst][i] = 0 + slot[a]   (a gradient read from the tape)      */
};
#define CTAMD_EXPR_MAX_INSNS 160
#define CTAMD_EXPR_MAX_SLOTS 32
#define CTAMD_EXPR_MAX_PORTS 8
typedef struct ctamd_expr_insn {
    uint8_t op, dst, a, b;
    float imm;
} ctamd_expr_insn;
/* Runs the program for every element of a [rows, cols] value.  prog, inputs and outputs are HOST
 * arrays (inputs / outputs hold device pointers), read before the call returns.  Full-shape
 * inputs and all outputs have rows * cols elements, row-vector inputs cols.  A slot must be
 * written before it is read.  status (one int32 on the device, cleared by the caller) is only
 * needed by programs with CTAMD_EX_DIVCHK.  An output must not alias an input that the program
 * reads after the store. */
int ctamd_expr_run_f32(const ctamd_expr_insn* prog, int n_insn, const float* const* inputs, int n_inputs,
                       float* const* outputs, int n_outputs, int32_t* status, size_t rows, size_t cols, void* stream);
/* A program that ctamd_expr_run_f32 has been handed `threshold` times is written out as a
 * straight-line HIP kernel, compiled for the device at run time (hiprtc; 20 - 200 ms, once per program
 * and math mode) and launched from then on in place of the interpreter: the same per-element
 * arithmetic from the same source text, so the same bits, without the interpreter's decoding and
 * with divisions by row vectors turned into multiplications by reciprocals formed once per thread.
 * threshold 0 switches compilation off, 1 compiles at first sight; default 2.  Operands that are not
 * 16-byte aligned, rows that are not a multiple of four, programs with row vectors over rows of fewer
 * than 512 elements, and launches that are being recorded into a graph before the program was
 * compiled, stay with the interpreter; so does a program whose compilation fails.  No counterpart in
 * the reference. */
int ctamd_set_expr_jit(int threshold);
int ctamd_expr_jit(void);
/* Programs compiled / that failed to compile, launches of compiled kernels / of the interpreter. */
void ctamd_expr_jit_stats(uint64_t* compiled, uint64_t* failed, uint64_t* compiled_launches, uint64_t* interpreted_launches);
/* Generates and compiles the kernel for `prog` in the current math mode without launching anything
 * (works without a GPU): columns = 1 for the access pattern of programs with row vectors, words = 128-bit
 * words per lane (1, 2 or 4).  text (may be null) receives up to cap bytes of the generated source,
 * code_bytes (may be null) the size of the code object. */
int ctamd_expr_jit_compile(const ctamd_expr_insn* prog, int n_insn, int columns, int words, char* text, size_t cap, size_t* code_bytes);

/* ----------------------------------------------------------------- backward arithmetic */
/* r[i] = v.  A 0-D gradient expanded to a shape: src/AutoDiff.cpp:579-592; also Tensor::zero()
 * / ones() src/Tensor.cpp:390-451. */
int ctamd_fill_f32(float* r, float v, size_t n, void* stream);
/* r[i] = v1[0] with v1 on the device (the tape's root gradient and loss gradients stay in HBM). */
int ctamd_fill_from_f32(float* r, const float* v1, size_t n, void* stream);
/* grad[i] += val[i] in place.  src/AutoDiff.cpp:1870-1878. */
int ctamd_accumulate_f32(float* grad, const float* val, size_t n, void* stream);
/* dx = g * (x > 0 ? 1 : 0) as a multiply, so g*0 keeps its sign and NaN/inf propagate.
 * src/AutoDiff.cpp:1334-1341, :1370. */
int ctamd_relu_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
/* s = sigmoid(x); dx = (s * (1 - s)) * g.  src/AutoDiff.cpp:1372-1383. */
int ctamd_sigmoid_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
/* t = tanh(x); dx = (1 - t*t) * g.  src/AutoDiff.cpp:1384-1398. */
int ctamd_tanh_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
/* dx = cos(x) * g; dx = (-sin(x)) * g.  src/AutoDiff.cpp:1399-1407, :1408-1416. */
int ctamd_sin_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
int ctamd_cos_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
/* The five gradients above with the gradient gathered so far added in the same pass:
 * dx[i] = acc[i] + term[i], the term rounded first - what the entry point above followed by
 * ctamd_accumulate_f32 leaves (src/AutoDiff.cpp:1870-1907), in 16 instead of 24 bytes per element.
 * For an operand that other operators use as well. */
int ctamd_relu_backward_acc_f32(const float* x, const float* g, const float* acc, float* dx, size_t n, void* stream);
int ctamd_sigmoid_backward_acc_f32(const float* x, const float* g, const float* acc, float* dx, size_t n, void* stream);
int ctamd_tanh_backward_acc_f32(const float* x, const float* g, const float* acc, float* dx, size_t n, void* stream);
int ctamd_sin_backward_acc_f32(const float* x, const float* g, const float* acc, float* dx, size_t n, void* stream);
int ctamd_cos_backward_acc_f32(const float* x, const float* g, const float* acc, float* dx, size_t n, void* stream);
/* out[i] = acc[i] + a[i] * b[i], the product rounded first: the Mul gradient term other * g
 * (src/AutoDiff.cpp:1234-1258) joining a gathered gradient (:1870-1907) in one pass. */
int ctamd_mul_acc_f32(const float* a, const float* b, const float* acc, float* out, size_t n, void* stream);
/* out[i] = acc[i] + a[i] / b[i], the quotient rounded first: Div's gradient term for its first
 * operand, g / b (src/AutoDiff.cpp:1285), joining a gathered gradient; b of a's shape, or (rowbcast) a
 * row vector [cols] under a [rows, cols]. */
int ctamd_div_acc_f32(const float* a, const float* b, const float* acc, float* out, size_t n, void* stream);
int ctamd_div_rowbcast_acc_f32(const float* a, const float* b, const float* acc, float* out, size_t rows, size_t cols,
                               void* stream);
/* dx = y * (g - sum_j g*y) per row (dim 1) or per column (dim 0), y the stored softmax output.
 * src/AutoDiff.cpp:1462-1472, :1473-1484. */
int ctamd_softmax_backward_rows_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols,
                                    void* stream);
int ctamd_softmax_backward_cols_f32(const float* y, const float* g, float* dx, size_t rows, size_t cols,
                                    void* stream);
/* dp = 0 + (((p - t) * 2) / n) * g[0]; dp = 0 + (sign(p - t) / n) * g[0]; g a 0-D device tensor.
 * src/AutoDiff.cpp:1491-1516, :1602-1642; the "0 +" is the tape adding the term to its zero-filled
 * gradient buffer (:1870-1907): a -0 term is stored as +0.  The cross-entropy gradients below
 * include it as well. */
int ctamd_mse_backward_f32(const float* p, const float* t, const float* g1, float* dp, size_t n, void* stream);
int ctamd_mae_backward_f32(const float* p, const float* t, const float* g1, float* dp, size_t n, void* stream);
/* The same two with the gradient gathered so far added in the same pass: dp[i] = acc[i] + term[i],
 * the term rounded first - what ctamd_mse/mae_backward_f32 followed by ctamd_accumulate_f32 leaves
 * (src/AutoDiff.cpp:1870-1907), in 16 instead of 24 bytes per element.  For a tensor that several
 * losses are taken of. */
int ctamd_mse_backward_acc_f32(const float* p, const float* t, const float* g1, const float* acc, float* dp, size_t n,
                               void* stream);
int ctamd_mae_backward_acc_f32(const float* p, const float* t, const float* g1, const float* acc, float* dp, size_t n,
                               void* stream);
/* dx = 0 + (softmax(x) - t) * g[0], gradient of the SUM-reduced loss.  src/AutoDiff.cpp:1546-1574.
 * The index form takes class indices (the reference throws there, :1569) and equals the one-hot
 * arithmetic with t = onehot(idx). */
int ctamd_cross_entropy_backward_onehot_f32(const float* x, const float* t, const float* g1, float* dx,
                                            size_t rows, size_t cols, void* stream);
int ctamd_cross_entropy_backward_index_f32(const float* x, const float* idx, const float* g1, float* dx,
                                           size_t rows, size_t cols, void* stream);
/* Gradients of the operators above that the reference declares without defining: sign(x) * g (sign(0)
 * = 0); g / (y * 2) with y = sqrt(x); (x * 2) * g; (1 + y * y) * g with y = tan(x); g * (x > 0 ? 1 :
 * slope).  exp's is y * g and log's g / x: ctamd_mul_f32 and ctamd_div_f32. */
int ctamd_abs_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
int ctamd_sqrt_backward_f32(const float* y, const float* g, float* dx, size_t n, void* stream);
int ctamd_square_backward_f32(const float* x, const float* g, float* dx, size_t n, void* stream);
int ctamd_tan_backward_f32(const float* y, const float* g, float* dx, size_t n, void* stream);
int ctamd_leaky_relu_backward_f32(const float* x, const float* g, float slope, float* dx, size_t n, void* stream);
/* db = ((-a) * g) / (b * b).  src/AutoDiff.cpp:1314.  (da = g / b is ctamd_div_f32, :1285.) */
int ctamd_div_backward_b_f32(const float* a, const float* b, const float* g, float* db, size_t n, void* stream);
/* The same for a row-vector divisor b[cols] under a[rows, cols] (the broadcast Div of this backend):
 * db_full[i, j] = ((-a[i, j]) * g[i, j]) / (b[j] * b[j]); the caller reduces it to b's shape. */
int ctamd_div_backward_b_rowbcast_f32(const float* a, const float* b, const float* g, float* db_full, size_t rows,
                                      size_t cols, void* stream);

/* ------------------------------------------- the MNIST demo's path (mnist/, "next" rows) */
/* dst[i] = src[i] / 255.0f, the loader's pixel normalisation (mnist/mnist_loader.cpp:35-41);
 * bit-exact. */
int ctamd_u8_to_unit_f32(const uint8_t* src, float* dst, size_t n, void* stream);
/* out[i, j] = (j == (int)labels[i]) ? 1 : 0, the demo's one-hot targets (mnist/mnist.cpp:72-78). */
int ctamd_onehot_f32(const float* labels, float* out, size_t rows, size_t classes, void* stream);
/* param[i] -= grad[i] * lr, product and difference rounded separately as in the reference's
 * binary (mnist/mnist.cpp:86-92; built without -O3/-march, CMakeLists.txt:56,65-86); bit-exact. */
int ctamd_sgd_step_f32(float* param, const float* grad, float lr, size_t n, void* stream);
/* The same update for every parameter of a model in one launch (update_parameters' loop over the
 * six tensors, mnist/mnist.cpp:86-92): params[t][i] -= (0 + grads[t][i]) * lr for t < tensors,
 * i < counts[t].  params, grads and counts are HOST arrays of device pointers / element counts,
 * read before the call returns.  "0 +" stands for reading the gradient out of the reference's tape,
 * whose buffers start zero-filled (src/AutoDiff.cpp:1870-1907): a -0 gradient counts as +0. */
int ctamd_sgd_step_multi_f32(float* const* params, const float* const* grads, const size_t* counts, int tensors, float lr,
                             void* stream);
/* count[0] = number of rows whose first maximum (strictly greater, starting from -1.0f at column
 * 0) is at column (int)labels[row]: calculate_accuracy (mnist/mnist.cpp:134-156) without its
 * division by the row count. */
int ctamd_count_correct_f32(const float* pred, const float* labels, int32_t* count, size_t rows, size_t classes,
                            void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CTORCH_AMD_H */
