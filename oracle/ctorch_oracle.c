/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the arithmetic of the reference's CPU-BASIC operators, of the host-inline
 * arithmetic in its Tensor front-end and of the per-operator gradient arithmetic in its tape.
 * Only tests, the smoke check and the CPU-baseline leg of the benchmark may load this file; the
 * shipped library never does.
 *
 * Every function names the reference lines it follows (paths relative to the reference root).
 * The reference library is built -O3 -march=native (CMakeLists.txt:65-86).  GCC 11 then treats
 * its sequential `acc += x*y` loops in two ways, and which one was found per loop by comparing
 * bits with the built library: loops it cannot vectorise (strided operands in MatMul and in the
 * column-wise softmax gradient, libm calls in CrossEntropy) get a fused multiply-add; loops over
 * contiguous memory (Dot, MSE, the row-wise softmax gradient) are vectorised as rounded products
 * that are then added in order, i.e. without fusion, except for a scalar tail of up to three
 * elements (see contiguous_mac).  Elementwise loops are never fused.  This
 * file is compiled with -ffp-contract=off and spells each fusion out with fmaf(), so that the
 * bits do not depend on this file's compiler.
 *
 * Pinning (tests/test_oracle_vs_ref.py, tests/test_oracle_golden.py, tests/test_oracle_math.py):
 * every function below is compared bit for bit with the real reference library where that has
 * been built (oracle/_ref), with the golden vectors written from it (tests/golden/), with the
 * known answers of the reference's own tests, and with closed forms / fp64 recomputation.
 * Functions the reference cannot express are marked "extension" and are pinned by the same-shape
 * reference kernel on hand-materialised operands or by fp64 mathematics:
 *   co_binary_rowbcast for Sub/Mul/Div, co_ce_bwd_index, co_colsum_f64.
 * co_expr_run (a per-element program of the operators above) is pinned opcode by opcode against
 * the whole-tensor functions here, which the reference pins, and on the config-5 chain against
 * co_expr; co_compare against the IEEE predicates the reference's plain C++ comparisons are
 * (tests/test_oracle_golden.py).  The functions for tensors that are not fp32 (co_cast_from_f32,
 * co_scalar_op_typed, co_softmax_f64) are pinned byte for byte against the reference's Tensor::to,
 * operator+ * / (float), zero / ones and softmax on double, int32, int64 and bool tensors
 * (tests/golden/typed.npz: edge conversions, wrapping sums and products, truncating scalars);
 * co_accumulate_typed against IEEE double addition and two's complement wrap.
 * The MNIST functions (co_u8_to_unit ... co_mnist_predict) are
 * pinned bit for bit against the reference's loader, demo functions and its own main()
 * (tests/test_oracle_vs_ref_mnist.py, tests/golden/mnist.npz).
 * co_adjust_grad_shape (the reference's whole gradient shape adjustment) is pinned bit for bit
 * against the reference through its public AutoDiff::backward(root, grad_output) on every shape pair
 * for which the reference stays inside its buffers (tests/test_oracle_vs_ref.py).
 * The methods the reference declares and never defines have no reference arithmetic to be in parity
 * with; their oracle functions are PINNED BY MATHEMATICS only (tests/test_oracle_math.py: numpy in
 * double, closed forms, brute force on tiny inputs, central differences for the gradients):
 *   co_unary_ext, co_unary_ext_bwd, co_reduce_dim, co_reduce_dim_bwd, co_log_softmax,
 *   co_log_softmax_bwd, co_broadcast_reduce.
 * Transcendentals call glibc libm (expf, logf, sinf, cosf) exactly as the reference does; their
 * values are whatever the installed glibc returns (2.35 in this image).
 */
#include "ctorch_oracle.h"

#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ forward: binary kernels */

/* src/kernels/CPU-BASIC/Add_BASIC_kernel.cpp:64-69 (same-shape branch) */
void co_add(const float* a, const float* b, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] + b[i];
}
/* src/kernels/CPU-BASIC/Sub_BASIC_kernel.cpp:58-60 */
void co_sub(const float* a, const float* b, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] - b[i];
}
/* src/kernels/CPU-BASIC/Mul_BASIC_kernel.cpp:59-61 */
void co_mul(const float* a, const float* b, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] * b[i];
}
/* src/kernels/CPU-BASIC/Div_BASIC_kernel.cpp:37-45: a zero divisor is logged, 0 is written and
 * then overwritten by the IEEE quotient, so the stored value is always a/b. */
void co_div(const float* a, const float* b, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] / b[i];
}
/* Add_BASIC_kernel.cpp:48-53: b.numel()==1, its single value is added to every element */
void co_add_scalar_tensor(const float* a, const float* b1, float* r, long n) {
    float v = b1[0];
    for (long i = 0; i < n; ++i) r[i] = a[i] + v;
}
/* Add_BASIC_kernel.cpp:54-63: a is [rows, cols], b is [cols]; r[i,j] = a[i,j] + b[j] */
void co_add_rowbcast(const float* a, const float* b, float* r, long rows, long cols) {
    for (long i = 0; i < rows; ++i)
        for (long j = 0; j < cols; ++j) r[i * cols + j] = a[i * cols + j] + b[j];
}
/* Extension: Add's row-broadcast convention for the other three operators (the reference throws
 * for Sub/Mul, Sub_BASIC_kernel.cpp:35-43 via Tensor.cpp:362-365, and reads out of bounds for
 * Div, Div_BASIC_kernel.cpp:18-20).  Equal by construction to the same-shape kernel applied to
 * a hand-materialised B[i,j] = b[j].  op: 0 add, 1 sub, 2 mul, 3 div. */
void co_binary_rowbcast(int op, const float* a, const float* b, float* r, long rows, long cols) {
    for (long i = 0; i < rows; ++i)
        for (long j = 0; j < cols; ++j) {
            float x = a[i * cols + j], y = b[j], z;
            switch (op) {
                case 0: z = x + y; break;
                case 1: z = x - y; break;
                case 2: z = x * y; break;
                default: z = x / y; break;
            }
            r[i * cols + j] = z;
        }
}

/* ------------------------------------------------------------------- forward: unary kernels */

/* src/kernels/CPU-BASIC/Neg_BASIC_kernel.cpp:26-28 */
void co_neg(const float* a, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = -a[i];
}
/* src/kernels/CPU-BASIC/ReLU_BASIC_kernel.cpp:23-25: std::max(0.0f, x) is (0.0f < x) ? x : 0.0f,
 * hence -0 -> +0 and NaN -> +0. */
void co_relu(const float* a, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = (0.0f < a[i]) ? a[i] : 0.0f;
}
/* src/kernels/CPU-BASIC/Sin_BASIC_kernel.cpp:24-26 */
void co_sin(const float* a, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = sinf(a[i]);
}
/* src/kernels/CPU-BASIC/Cos_BASIC_kernel.cpp:23-25 */
void co_cos(const float* a, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = cosf(a[i]);
}
/* src/kernels/CPU-BASIC/Tanh_BASIC_kernel.cpp:24-28 */
void co_tanh(const float* a, float* r, long n) {
    for (long i = 0; i < n; ++i) {
        float ep = expf(a[i]);
        float en = expf(-a[i]);
        r[i] = (ep - en) / (ep + en);
    }
}
/* src/kernels/CPU-BASIC/Sigmoid_BASIC_kernel.cpp:24-26 */
void co_sigmoid(const float* a, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = 1.0f / (1.0f + expf(-a[i]));
}

/* src/Tensor.cpp:1676-1684 (1-D), :1713-1727 (dim 1), :1728-1744 (dim 0): the live softmax;
 * with guard_zero_sum it is the registered kernel instead
 * (src/kernels/CPU-BASIC/Softmax_BASIC_kernel.cpp:47-64, :72-93, which only has dim 1).
 * A 1-D input is passed as rows = 1, dim = 1. */
void co_softmax(const float* x, float* y, long rows, long cols, int dim, int guard_zero_sum) {
    if (dim == 1) {
        for (long i = 0; i < rows; ++i) {
            const float* in = x + i * cols;
            float* out = y + i * cols;
            float m = in[0];
            for (long j = 1; j < cols; ++j)
                if (in[j] > m) m = in[j];
            float s = 0.0f;
            for (long j = 0; j < cols; ++j) {
                float e = expf(in[j] - m);
                out[j] = e;
                s += e;
            }
            if (!guard_zero_sum || s > 0.0f)
                for (long j = 0; j < cols; ++j) out[j] /= s;
        }
    } else {
        for (long j = 0; j < cols; ++j) {
            float m = x[j];
            for (long i = 1; i < rows; ++i)
                if (x[i * cols + j] > m) m = x[i * cols + j];
            float s = 0.0f;
            for (long i = 0; i < rows; ++i) {
                float e = expf(x[i * cols + j] - m);
                y[i * cols + j] = e;
                s += e;
            }
            for (long i = 0; i < rows; ++i) y[i * cols + j] /= s;
        }
    }
}

/* src/kernels/CPU-BASIC/MatMul_BASIC_kernel.cpp:42-54: i-j-l order, stride-aware operands, one
 * fp32 accumulator per output, fused multiply-add in the built reference. */
void co_matmul(const float* a, long as0, long as1, const float* b, long bs0, long bs1, float* c,
               long m, long n, long k) {
    for (long i = 0; i < m; ++i)
        for (long j = 0; j < n; ++j) {
            float s = 0.0f;
            for (long l = 0; l < k; ++l) s = fmaf(a[i * as0 + l * as1], b[l * bs0 + j * bs1], s);
            c[i * n + j] = s;
        }
}

/* The shape GCC 11 -O3 gives a contiguous `acc += x[i]*y[i]` loop on AVX2/AVX-512 hosts that
 * prefer 256-bit vectors (found by comparing bits with the built reference for every length
 * 1..40 and several longer ones): blocks of 8 rounded products added in order, then one block
 * of 4 if at least 4 elements remain, then a scalar tail of at most 3 fused multiply-adds. */
static float contiguous_mac(const float* x, const float* y, long n, float s) {
    long i = 0, main_end = n / 8 * 8;
    for (; i < main_end; ++i) {
        float p = x[i] * y[i];
        s += p;
    }
    if (n - i >= 4)
        for (long e = i + 4; i < e; ++i) {
            float p = x[i] * y[i];
            s += p;
        }
    for (; i < n; ++i) s = fmaf(x[i], y[i], s);
    return s;
}

/* src/kernels/CPU-BASIC/Dot_BASIC_kernel.cpp:38-41 */
float co_dot(const float* a, const float* b, long n) { return contiguous_mac(a, b, n, 0.0f); }

/* src/kernels/CPU-BASIC/MSE_BASIC_kernel.cpp:35-41: the same loop shape over d = a - b */
float co_mse(const float* a, const float* b, long n) {
    float s = 0.0f;
    long i = 0, main_end = n / 8 * 8;
    for (; i < main_end; ++i) {
        float d = a[i] - b[i];
        float q = d * d;
        s += q;
    }
    if (n - i >= 4)
        for (long e = i + 4; i < e; ++i) {
            float d = a[i] - b[i];
            float q = d * d;
            s += q;
        }
    for (; i < n; ++i) {
        float d = a[i] - b[i];
        s = fmaf(d, d, s);
    }
    return s / (float)(size_t)n;
}
/* src/kernels/CPU-BASIC/MAE_BASIC_kernel.cpp:35-41 */
float co_mae(const float* a, const float* b, long n) {
    float s = 0.0f;
    for (long i = 0; i < n; ++i) {
        float d = a[i] - b[i];
        s += fabsf(d);
    }
    return s / (float)(size_t)n;
}

static float row_max(const float* x, long cols) {
    float m = x[0];
    for (long j = 1; j < cols; ++j)
        if (x[j] > m) m = x[j];
    return m;
}
static float row_expsum(const float* x, long cols, float m) {
    float s = 0.0f;
    for (long j = 0; j < cols; ++j) s += expf(x[j] - m);
    return s;
}

/* src/kernels/CPU-BASIC/CrossEntropy_BASIC_kernel.cpp:41-66 (2-D one-hot; the 1-D form :67-82 is
 * rows = 1): the loss is SUMMED over rows, never averaged; std::max(pred, 1e-10f) is
 * (pred < 1e-10f) ? 1e-10f : pred; `ce -= t * log(pred)` is one fused multiply-add. */
float co_ce_onehot(const float* x, const float* t, long rows, long cols) {
    float ce = 0.0f;
    for (long i = 0; i < rows; ++i) {
        const float* xi = x + i * cols;
        float m = row_max(xi, cols);
        float s = row_expsum(xi, cols, m);
        for (long j = 0; j < cols; ++j) {
            float p = expf(xi[j] - m) / s;
            p = (p < 1e-10f) ? 1e-10f : p;
            ce = fmaf(-t[i * cols + j], logf(p), ce);
        }
    }
    return ce;
}
/* CrossEntropy_BASIC_kernel.cpp:88-120 (class indices held as floats, truncated toward zero).
 * Returns 0 and the summed loss, or -1 when an index is out of range (the reference then returns
 * an empty Tensor, :96-100). */
int co_ce_index(const float* x, const float* idx, long rows, long cols, float* out) {
    float ce = 0.0f;
    for (long i = 0; i < rows; ++i) {
        int c = (int)idx[i];
        if (c < 0 || c >= (int)cols) return -1;
        const float* xi = x + i * cols;
        float m = row_max(xi, cols);
        float s = row_expsum(xi, cols, m);
        float p = expf(xi[c] - m) / s;
        p = (p < 1e-10f) ? 1e-10f : p;
        ce -= logf(p);
    }
    *out = ce;
    return 0;
}

/* --------------------------------------------------- forward: host-inline Tensor arithmetic */

/* src/Tensor.cpp:644-647 */
float co_sum(const float* a, long n) {
    float s = 0.0f;
    for (long i = 0; i < n; ++i) s += a[i];
    return s;
}
/* src/Tensor.cpp:862-868 */
void co_scalar_add(const float* a, float s, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] + s;
}
/* src/Tensor.cpp:759-765 */
void co_scalar_mul(const float* a, float s, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] * s;
}
/* src/Tensor.cpp:925-931 */
void co_scalar_div(const float* a, float s, float* r, long n) {
    for (long i = 0; i < n; ++i) r[i] = a[i] / s;
}

/* ----------------------------------------------------------------------- backward arithmetic */

/* src/AutoDiff.cpp:579-592: a 0-D gradient is expanded to the target shape */
void co_fill(float* r, float v, long n) {
    for (long i = 0; i < n; ++i) r[i] = v;
}
/* src/AutoDiff.cpp:1870-1878: in-place grad[i] += val[i] */
void co_accumulate(float* grad, const float* val, long n) {
    for (long i = 0; i < n; ++i) grad[i] += val[i];
}
/* src/AutoDiff.cpp:706-757 as it behaves for g [rows, cols] -> target [cols]: the result is
 * zeroed and then receives g's leading-index-0 slice, 0.0f + g[0, j] (it does not sum over rows;
 * the reference's own test expects that: src/tests/test_tensor_grad.cpp:132-138). */
void co_adjust_row0(const float* g, float* r, long rows, long cols) {
    (void)rows;
    for (long j = 0; j < cols; ++j) r[j] = 0.0f + g[j];
}
/* Extension: the mathematically complete gradient of a row-broadcast operand, sum over rows,
 * accumulated in double as the arbiter for the device column-sum kernel. */
void co_colsum_f64(const float* g, double* r, long rows, long cols) {
    for (long j = 0; j < cols; ++j) r[j] = 0.0;
    for (long i = 0; i < rows; ++i)
        for (long j = 0; j < cols; ++j) r[j] += (double)g[i * cols + j];
}
/* src/AutoDiff.cpp:1334-1341 + :1370: mask = x>0 ? 1 : 0, then node_grad * mask (Mul kernel) */
void co_relu_bwd(const float* x, const float* g, float* dx, long n) {
    for (long i = 0; i < n; ++i) {
        float mask = (x[i] > 0.0f) ? 1.0f : 0.0f;
        dx[i] = g[i] * mask;
    }
}
/* src/AutoDiff.cpp:1372-1383: s = sigmoid(x); (s * (1.0f - s)) * g */
void co_sigmoid_bwd(const float* x, const float* g, float* dx, long n) {
    for (long i = 0; i < n; ++i) {
        float s = 1.0f / (1.0f + expf(-x[i]));
        float om = 1.0f - s;
        float p = s * om;
        dx[i] = p * g[i];
    }
}
/* src/AutoDiff.cpp:1384-1398: t = tanh(x); (1.0f - t*t) * g */
void co_tanh_bwd(const float* x, const float* g, float* dx, long n) {
    for (long i = 0; i < n; ++i) {
        float ep = expf(x[i]);
        float en = expf(-x[i]);
        float t = (ep - en) / (ep + en);
        float tt = t * t;
        float om = 1.0f - tt;
        dx[i] = om * g[i];
    }
}
/* src/AutoDiff.cpp:1399-1407: cos(x) * g */
void co_sin_bwd(const float* x, const float* g, float* dx, long n) {
    for (long i = 0; i < n; ++i) dx[i] = cosf(x[i]) * g[i];
}
/* src/AutoDiff.cpp:1408-1416: (-sin(x)) * g */
void co_cos_bwd(const float* x, const float* g, float* dx, long n) {
    for (long i = 0; i < n; ++i) dx[i] = (-sinf(x[i])) * g[i];
}
/* src/AutoDiff.cpp:1441-1446 (1-D), :1462-1472 (dim 1), :1473-1484 (dim 0): uses the stored
 * output y; dx = y * (g - dot).  The row-wise dot walks contiguous memory and is compiled like
 * Dot above (contiguous_mac); the column-wise dot is strided and is compiled
 * as a fused multiply-add chain.  Both were checked against the built reference. */
void co_softmax_bwd(const float* y, const float* g, float* dx, long rows, long cols, int dim) {
    if (dim == 1) {
        for (long i = 0; i < rows; ++i) {
            float d = 0.0f;
            d = contiguous_mac(g + i * cols, y + i * cols, cols, 0.0f);
            for (long j = 0; j < cols; ++j) dx[i * cols + j] = y[i * cols + j] * (g[i * cols + j] - d);
        }
    } else {
        for (long j = 0; j < cols; ++j) {
            float d = 0.0f;
            for (long i = 0; i < rows; ++i) d = fmaf(g[i * cols + j], y[i * cols + j], d);
            for (long i = 0; i < rows; ++i) dx[i * cols + j] = y[i * cols + j] * (g[i * cols + j] - d);
        }
    }
}
/* src/AutoDiff.cpp:1491-1516: (((p - t) * 2.0f) / float(n)) * g with g the 0-D upstream value */
void co_mse_bwd(const float* p, const float* t, float g, float* dp, long n) {
    float fn = (float)(size_t)n;
    for (long i = 0; i < n; ++i) {
        float d = p[i] - t[i];
        float d2 = d * 2.0f;
        float q = d2 / fn;
        dp[i] = q * g;
    }
}
/* src/AutoDiff.cpp:1602-1642: (sign(p - t) / float(n)) * g, sign in {1, -1, 0} */
void co_mae_bwd(const float* p, const float* t, float g, float* dp, long n) {
    float fn = (float)(size_t)n;
    for (long i = 0; i < n; ++i) {
        float d = p[i] - t[i];
        float s = (d > 0.0f) ? 1.0f : ((d < 0.0f) ? -1.0f : 0.0f);
        float q = s / fn;
        dp[i] = q * g;
    }
}
/* src/AutoDiff.cpp:1546-1574: row softmax recomputed (no stored sum of stored exps: the sum and
 * the numerators are separate expf passes), minus the one-hot target (Sub kernel), times the
 * upstream scalar (scalar Mul).  Gradient of the SUM-reduced loss. */
void co_ce_bwd_onehot(const float* x, const float* t, float g, float* dx, long rows, long cols) {
    for (long i = 0; i < rows; ++i) {
        const float* xi = x + i * cols;
        float m = row_max(xi, cols);
        float s = row_expsum(xi, cols, m);
        for (long j = 0; j < cols; ++j) {
            float sm = expf(xi[j] - m) / s;
            float d = sm - t[i * cols + j];
            dx[i * cols + j] = d * g;
        }
    }
}
/* Extension: the same arithmetic with class-index targets (the reference throws here,
 * AutoDiff.cpp:1569 through the Sub broadcast): target is 1.0f at idx[i], 0.0f elsewhere. */
void co_ce_bwd_index(const float* x, const float* idx, float g, float* dx, long rows, long cols) {
    for (long i = 0; i < rows; ++i) {
        const float* xi = x + i * cols;
        int c = (int)idx[i];
        float m = row_max(xi, cols);
        float s = row_expsum(xi, cols, m);
        for (long j = 0; j < cols; ++j) {
            float sm = expf(xi[j] - m) / s;
            float d = sm - ((j == c) ? 1.0f : 0.0f);
            dx[i * cols + j] = d * g;
        }
    }
}
/* src/AutoDiff.cpp:1285: node_grad / b */
void co_div_bwd_a(const float* g, const float* b, float* da, long n) {
    for (long i = 0; i < n; ++i) da[i] = g[i] / b[i];
}
/* src/AutoDiff.cpp:1314: ((-a) * g) / (b * b) - Neg, Mul, Mul, Div in that order */
void co_div_bwd_b(const float* a, const float* b, const float* g, float* db, long n) {
    for (long i = 0; i < n; ++i) {
        float na = -a[i];
        float num = na * g[i];
        float den = b[i] * b[i];
        db[i] = num / den;
    }
}
/* src/AutoDiff.cpp:1267-1279: the divisor scan that makes Div's backward throw */
int co_any_abs_lt_eps(const float* b, long n) {
    for (long i = 0; i < n; ++i)
        if (fabsf(b[i]) < FLT_EPSILON) return 1;
    return 0;
}

/* --------------------------------------------------------------------------- configurations */

static float* falloc(long n) {
    float* p = (float*)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
    if (!p) abort();
    return p;
}

/* c = a*b + 5.0f; d = relu(c); s = d.sum(); s.backward().  Forward: Mul_BASIC_kernel,
 * Tensor::operator+(float) (src/Tensor.cpp:855-910), ReLU_BASIC_kernel, Tensor::sum.  Backward
 * (src/AutoDiff.cpp:1080-1924): root grad 1 -> Sum: fill (1850-1855) -> ReLU: g*mask -> Add with
 * the taped 0-D scalar: pass-through -> Mul: other * g (1234-1258); every edge lands with
 * grad += val on a zeroed gradient (1870-1878). */
void co_chain(const float* a, const float* b, long n, float* s, float* ga, float* gb) {
    float* c = falloc(n);
    float* d = falloc(n);
    float* g = falloc(n);
    float* v = falloc(n);
    co_mul(a, b, c, n);
    co_scalar_add(c, 5.0f, c, n);
    co_relu(c, d, n);
    *s = co_sum(d, n);
    /* grad(d) = 0 + fill(1) */
    co_fill(g, 0.0f, n);
    co_fill(v, 1.0f, n);
    co_accumulate(g, v, n);
    /* grad(c) = 0 + grad(d) * mask(c) */
    co_relu_bwd(c, g, v, n);
    co_fill(g, 0.0f, n);
    co_accumulate(g, v, n);
    /* grad(a*b) = 0 + grad(c)   (Add branch) */
    memcpy(v, g, (size_t)n * sizeof(float));
    co_fill(g, 0.0f, n);
    co_accumulate(g, v, n);
    /* grad(a) = 0 + b * g ; grad(b) = 0 + a * g */
    co_mul(b, g, v, n);
    co_fill(ga, 0.0f, n);
    co_accumulate(ga, v, n);
    co_mul(a, g, v, n);
    co_fill(gb, 0.0f, n);
    co_accumulate(gb, v, n);
    free(c);
    free(d);
    free(g);
    free(v);
}

static void zero_plus(float* dst, const float* val, long n) {
    for (long i = 0; i < n; ++i) dst[i] = 0.0f + val[i];
}

/* logits = relu(x*W1 + b1)*W2 + b2; loss = CE_sum(logits, onehot); backward
 * (mnist/mnist.cpp:38-42,66-75 with one hidden layer).  MatMul backward is
 * dA = g.matmul(B.t()), dB = A.t().matmul(g) through the strided kernel
 * (src/AutoDiff.cpp:1692-1704, :1808-1810).  Bias gradients: strict_row0 = 1 reproduces the
 * reference (row 0 of the upstream gradient), 0 gives the column sum rounded from double. */
void co_mlp_step(const float* x, long B, long I, const float* W1, const float* b1, long H,
                 const float* W2, const float* b2, long C, const float* onehot, int strict_row0,
                 float* loss, float* logits, float* gW1, float* gb1, float* gW2, float* gb2) {
    float* z1 = falloc(B * H);
    float* a1 = falloc(B * H);
    float* h = falloc(B * H);
    float* z2 = falloc(B * C);
    float* gl = falloc(B * C);
    float* gh = falloc(B * H);
    float* ga1 = falloc(B * H);
    float* tmp = falloc(B * H > I * H ? B * H : I * H);
    double* cs = (double*)malloc((size_t)(H > C ? H : C) * sizeof(double));
    co_matmul(x, I, 1, W1, H, 1, z1, B, H, I);
    co_add_rowbcast(z1, b1, a1, B, H);
    co_relu(a1, h, B * H);
    co_matmul(h, H, 1, W2, C, 1, z2, B, C, H);
    co_add_rowbcast(z2, b2, logits, B, C);
    *loss = co_ce_onehot(logits, onehot, B, C);
    /* grad(logits) = 0 + (softmax - onehot) * 1.0f */
    co_ce_bwd_onehot(logits, onehot, 1.0f, tmp, B, C);
    zero_plus(gl, tmp, B * C);
    /* Add: grad(z2) = 0 + gl; grad(b2) = 0 + adjust(gl) */
    if (strict_row0) {
        co_adjust_row0(gl, tmp, B, C);
        zero_plus(gb2, tmp, C);
    } else {
        co_colsum_f64(gl, cs, B, C);
        for (long j = 0; j < C; ++j) gb2[j] = (float)cs[j];
    }
    /* MatMul: grad(h) = gl * W2^T ; grad(W2) = h^T * gl */
    co_matmul(gl, C, 1, W2, 1, C, tmp, B, H, C);
    zero_plus(gh, tmp, B * H);
    co_matmul(h, 1, H, gl, C, 1, tmp, H, C, B);
    zero_plus(gW2, tmp, H * C);
    /* ReLU: grad(a1) = 0 + gh * mask(a1) */
    co_relu_bwd(a1, gh, tmp, B * H);
    zero_plus(ga1, tmp, B * H);
    if (strict_row0) {
        co_adjust_row0(ga1, tmp, B, H);
        zero_plus(gb1, tmp, H);
    } else {
        co_colsum_f64(ga1, cs, B, H);
        for (long j = 0; j < H; ++j) gb1[j] = (float)cs[j];
    }
    /* MatMul: grad(W1) = x^T * grad(z1) (grad(z1) = 0 + ga1 = ga1) */
    co_matmul(x, 1, I, ga1, H, 1, tmp, I, H, B);
    zero_plus(gW1, tmp, I * H);
    free(z1);
    free(a1);
    free(h);
    free(z2);
    free(gl);
    free(gh);
    free(ga1);
    free(tmp);
    free(cs);
}

/* ---- the MNIST demo's path: loader arithmetic, targets, optimiser step, accuracy, train loop.
 * mnist/mnist.cpp and mnist/mnist_loader.cpp are built by the reference WITHOUT the library's
 * -O3 -march=native (CMakeLists.txt:56, :65-86 set those on the CTorch target only), so their own
 * arithmetic is plain IEEE, one rounding per operation: no FMA in the optimiser update. */

/* mnist/mnist_loader.cpp:35-41: pixel / 255.0f */
void co_u8_to_unit(const unsigned char* src, float* dst, long n) {
    for (long i = 0; i < n; ++i) dst[i] = (float)src[i] / 255.0f;
}

/* mnist/mnist.cpp:72-78: out[i, j] = (j == int(label_i)) ? 1 : 0 */
void co_onehot(const float* labels, float* out, long rows, long classes) {
    for (long i = 0; i < rows; ++i) {
        int lab = (int)labels[i];
        for (long j = 0; j < classes; ++j) out[i * classes + j] = (j == lab) ? 1.0f : 0.0f;
    }
}

/* mnist/mnist.cpp:86-92: p[i] -= g[i] * lr, product rounded, then the difference rounded */
void co_sgd_step(float* p, const float* g, float lr, long n) {
    for (long i = 0; i < n; ++i) {
        float step = g[i] * lr;
        p[i] = p[i] - step;
    }
}

/* mnist/mnist.cpp:134-156: per row the first index whose value exceeds every earlier one,
 * starting from -1.0f at index 0; counted when it equals int(label). */
long co_count_correct(const float* pred, const float* labels, long rows, long classes) {
    long correct = 0;
    for (long i = 0; i < rows; ++i) {
        int best = 0;
        float mx = -1.0f;
        for (long j = 0; j < classes; ++j) {
            float v = pred[i * classes + j];
            if (v > mx) {
                mx = v;
                best = (int)j;
            }
        }
        if (best == (int)labels[i]) ++correct;
    }
    return correct;
}

/* mnist/mnist.cpp:15-93 (the model and train_step) and :244-265 (the batch loop), `steps`
 * consecutive batches of `batch` rows, batch index = step % (n_images / batch) (:233, :252):
 *   logits = relu(relu(x W1 + b1) W2 + b2) W3 + b3; loss = CE_sum(logits, onehot); backward;
 *   every parameter p -= grad * lr.
 * Two properties of the reference's tape decide the bits (both reproduced when the flag is set,
 * both pinned against the built reference in tests/test_oracle_vs_ref.py):
 *   strict_row0     the gradient of a bias is row 0 of the upstream gradient
 *                   (src/AutoDiff.cpp:690-757), not the column sum;
 *   stale_snapshot  a leaf's node holds the deep copy made when the leaf was first seen
 *                   (src/AutoDiff.cpp:265-278 returns early for a known id) and MatMul's backward
 *                   reads operands from the nodes (:1692-1704), so the gradients that flow back
 *                   through W2 and W3 use the weights of the FIRST step, while the forward pass
 *                   and the weight gradients themselves use live values.
 * With both flags 0 this is plain SGD with column-sum bias gradients (rounded from double).
 * Parameters are updated in place; losses[s] is the loss of step s. */
void co_mnist_train(const float* images, const float* labels, long n_images, long I, long H1, long H2,
                    long C, float* W1, float* b1, float* W2, float* b2, float* W3, float* b3, long batch,
                    long steps, float lr, int strict_row0, int stale_snapshot, float* losses) {
    const long B = batch, nb = n_images / batch;
    long big = B * I;
    if (I * H1 > big) big = I * H1;
    if (H1 * H2 > big) big = H1 * H2;
    if (B * H1 > big) big = B * H1;
    float *z = falloc(B * H1), *a1 = falloc(B * H1), *h1 = falloc(B * H1), *a2 = falloc(B * H2),
          *h2 = falloc(B * H2), *logits = falloc(B * C), *oh = falloc(B * C), *gl = falloc(B * C),
          *gh2 = falloc(B * H2), *ga2 = falloc(B * H2), *gh1 = falloc(B * H1), *ga1 = falloc(B * H1),
          *tmp = falloc(big), *gW1 = falloc(I * H1), *gW2 = falloc(H1 * H2), *gW3 = falloc(H2 * C),
          *gb1 = falloc(H1), *gb2 = falloc(H2), *gb3 = falloc(C), *S2 = falloc(H1 * H2), *S3 = falloc(H2 * C);
    long widest = H1 > H2 ? H1 : H2;
    if (C > widest) widest = C;
    double* cs = (double*)malloc((size_t)widest * sizeof(double));
    memcpy(S2, W2, (size_t)(H1 * H2) * sizeof(float));
    memcpy(S3, W3, (size_t)(H2 * C) * sizeof(float));
    for (long s = 0; s < steps; ++s) {
        const long b = nb > 0 ? s % nb : 0;
        const float* x = images + b * B * I;
        const float* y = labels + b * B;
        co_matmul(x, I, 1, W1, H1, 1, z, B, H1, I);
        co_add_rowbcast(z, b1, a1, B, H1);
        co_relu(a1, h1, B * H1);
        co_matmul(h1, H1, 1, W2, H2, 1, z, B, H2, H1);
        co_add_rowbcast(z, b2, a2, B, H2);
        co_relu(a2, h2, B * H2);
        co_matmul(h2, H2, 1, W3, C, 1, z, B, C, H2);
        co_add_rowbcast(z, b3, logits, B, C);
        co_onehot(y, oh, B, C);
        losses[s] = co_ce_onehot(logits, oh, B, C);
        const float* B2 = stale_snapshot ? S2 : W2;
        const float* B3 = stale_snapshot ? S3 : W3;
        /* every gradient below is "zero-filled, then += value" (src/AutoDiff.cpp:1870-1907) */
        co_ce_bwd_onehot(logits, oh, 1.0f, tmp, B, C);
        zero_plus(gl, tmp, B * C);
#define CO_BIAS_GRAD(g, out, cols)                                        \
    if (strict_row0) {                                                     \
        co_adjust_row0(g, tmp, B, cols);                                   \
        zero_plus(out, tmp, cols);                                         \
    } else {                                                               \
        co_colsum_f64(g, cs, B, cols);                                     \
        for (long j = 0; j < cols; ++j) out[j] = (float)cs[j];             \
    }
        CO_BIAS_GRAD(gl, gb3, C)
        co_matmul(gl, C, 1, B3, 1, C, tmp, B, H2, C);          /* grad(h2) = gl . W3^T */
        zero_plus(gh2, tmp, B * H2);
        co_matmul(h2, 1, H2, gl, C, 1, tmp, H2, C, B);         /* grad(W3) = h2^T . gl */
        zero_plus(gW3, tmp, H2 * C);
        co_relu_bwd(a2, gh2, tmp, B * H2);
        zero_plus(ga2, tmp, B * H2);
        CO_BIAS_GRAD(ga2, gb2, H2)
        co_matmul(ga2, H2, 1, B2, 1, H2, tmp, B, H1, H2);      /* grad(h1) = ga2 . W2^T */
        zero_plus(gh1, tmp, B * H1);
        co_matmul(h1, 1, H1, ga2, H2, 1, tmp, H1, H2, B);      /* grad(W2) = h1^T . ga2 */
        zero_plus(gW2, tmp, H1 * H2);
        co_relu_bwd(a1, gh1, tmp, B * H1);
        zero_plus(ga1, tmp, B * H1);
        CO_BIAS_GRAD(ga1, gb1, H1)
        co_matmul(x, 1, I, ga1, H1, 1, tmp, I, H1, B);         /* grad(W1) = x^T . ga1 */
        zero_plus(gW1, tmp, I * H1);
#undef CO_BIAS_GRAD
        co_sgd_step(W1, gW1, lr, I * H1);
        co_sgd_step(b1, gb1, lr, H1);
        co_sgd_step(W2, gW2, lr, H1 * H2);
        co_sgd_step(b2, gb2, lr, H2);
        co_sgd_step(W3, gW3, lr, H2 * C);
        co_sgd_step(b3, gb3, lr, C);
    }
    free(z); free(a1); free(h1); free(a2); free(h2); free(logits); free(oh); free(gl); free(gh2);
    free(ga2); free(gh1); free(ga1); free(tmp); free(gW1); free(gW2); free(gW3); free(gb1); free(gb2);
    free(gb3); free(S2); free(S3); free(cs);
}

/* The demo's forward pass for prediction (mnist/mnist.cpp:95-130): logits, then a row softmax. */
void co_mnist_predict(const float* x, long B, long I, long H1, long H2, long C, const float* W1,
                      const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
                      float* probs) {
    float *z = falloc(B * (H1 > H2 ? H1 : H2)), *h1 = falloc(B * H1), *h2 = falloc(B * H2), *lg = falloc(B * C);
    co_matmul(x, I, 1, W1, H1, 1, z, B, H1, I);
    co_add_rowbcast(z, b1, h1, B, H1);
    co_relu(h1, h1, B * H1);
    co_matmul(h1, H1, 1, W2, H2, 1, z, B, H2, H1);
    co_add_rowbcast(z, b2, h2, B, H2);
    co_relu(h2, h2, B * H2);
    co_matmul(h2, H2, 1, W3, C, 1, z, B, C, H2);
    co_add_rowbcast(z, b3, lg, B, C);
    co_softmax(lg, probs, B, C, 1, 0);
    free(z); free(h1); free(h2); free(lg);
}

/* Y = sigmoid(X / R) - tanh(X) * sin(X) + cos(-X); L = mse(Y,T) + mae(Y,T); one backward.
 * R is a full [rows, cols] operand here (the reference's Div needs equal shapes).  The edge
 * order follows the reference's reversed depth-first order (src/AutoDiff.cpp:1138-1153); it
 * only matters for X, which receives four contributions: they are added in the order
 * cos-branch, sin, tanh, div when traversed from L. The exact order of those additions is
 * pinned against the real reference in tests/test_oracle_vs_ref.py. */
void co_expr(const float* X, const float* R, const float* T, long rows, long cols, float* Y,
             float* mse, float* mae, float* gX, float* gR) {
    long n = rows * cols;
    float *q = falloc(n), *s1 = falloc(n), *th = falloc(n), *sn = falloc(n), *m = falloc(n),
          *d1 = falloc(n), *ng = falloc(n), *cs = falloc(n), *gY = falloc(n), *v = falloc(n),
          *gd1 = falloc(n), *gcs = falloc(n), *gs1 = falloc(n), *gm = falloc(n), *gq = falloc(n),
          *gth = falloc(n), *gsn = falloc(n), *gng = falloc(n);
    co_div(X, R, q, n);
    co_sigmoid(q, s1, n);
    co_tanh(X, th, n);
    co_sin(X, sn, n);
    co_mul(th, sn, m, n);
    co_sub(s1, m, d1, n);
    co_neg(X, ng, n);
    co_cos(ng, cs, n);
    co_add(d1, cs, Y, n);
    *mse = co_mse(Y, T, n);
    *mae = co_mae(Y, T, n);
    /* L = l1 + l2: both losses get 0 + 1.0f; the order in which their gradients reach Y is
     * part of what the comparison with the real reference pins (contributions are summed in
     * fp32, and a+b is commutative, so two terms give the same bits either way). */
    co_fill(gY, 0.0f, n);
    co_mse_bwd(Y, T, 1.0f, v, n);
    float* v2 = falloc(n);
    co_mae_bwd(Y, T, 1.0f, v2, n);
    /* order decided against the reference: see co_expr_order in the tests */
    co_accumulate(gY, v2, n);
    co_accumulate(gY, v, n);
    free(v2);
    /* Add: d1 and cs get gY */
    zero_plus(gd1, gY, n);
    zero_plus(gcs, gY, n);
    /* Sub: s1 gets gd1, m gets -gd1 */
    zero_plus(gs1, gd1, n);
    co_neg(gd1, v, n);
    zero_plus(gm, v, n);
    /* Mul: th gets sn*gm, sn gets th*gm */
    co_mul(sn, gm, v, n);
    zero_plus(gth, v, n);
    co_mul(th, gm, v, n);
    zero_plus(gsn, v, n);
    /* Sigmoid: q gets sigmoid'(q)*gs1 */
    co_sigmoid_bwd(q, gs1, v, n);
    zero_plus(gq, v, n);
    /* Cos: ng gets (-sin(ng))*gcs ; Neg: X gets -gng */
    co_cos_bwd(ng, gcs, v, n);
    zero_plus(gng, v, n);
    /* Div: R gets ((-X)*gq)/(R*R) */
    co_div_bwd_b(X, R, gq, v, n);
    zero_plus(gR, v, n);
    /* X: contributions in tape order (pinned by test) */
    co_fill(gX, 0.0f, n);
    co_neg(gng, v, n);
    co_accumulate(gX, v, n);
    co_sin_bwd(X, gsn, v, n);
    co_accumulate(gX, v, n);
    co_tanh_bwd(X, gth, v, n);
    co_accumulate(gX, v, n);
    co_div_bwd_a(gq, R, v, n);
    co_accumulate(gX, v, n);
    free(q); free(s1); free(th); free(sn); free(m); free(d1); free(ng); free(cs); free(gY);
    free(v); free(gd1); free(gcs); free(gs1); free(gm); free(gq); free(gth); free(gsn); free(gng);
}

/* ------------------------------------------------------------------------ comparisons */

/* src/Tensor.cpp:985-1116 (tensor against float) and :1119-1309 (tensor against tensor of the same
 * shape): one bool per element.  cmp: 0 '>', 1 '<', 2 '==', 3 '>=', 4 '<=', 5 '!='.  b == NULL
 * compares with s.  (operator!=(const Tensor&) is declared in the reference's Tensor.h and never
 * defined; it is stated here as the negation of ==.) */
void co_compare(int cmp, const float* a, const float* b, float s, unsigned char* out, long n) {
    for (long i = 0; i < n; ++i) {
        const float x = a[i], y = b ? b[i] : s;
        out[i] = (unsigned char)(cmp == 0 ? x > y : cmp == 1 ? x < y : cmp == 2 ? x == y : cmp == 3 ? x >= y : cmp == 4 ? x <= y : x != y);
    }
}

/* ------------------------------------------------------------- tensors that are not fp32 */
/* dtype codes are the order of enum DType (include/Ctools.h:163-169): 0 float, 1 double, 2 int32,
 * 3 int64, 4 bool (one byte). */

/* static_cast<int32_t / int64_t>(float) as the reference's x86-64 build computes it (cvttss2si and
 * its vector forms): truncation toward zero, and the "integer indefinite" value 0x80...0 for NaN
 * and for values out of range - which C leaves undefined, so it is spelled out here. */
static int32_t f32_to_i32(float x) { return (x >= -2147483648.0f && x < 2147483648.0f) ? (int32_t)x : INT32_MIN; }
static int64_t f32_to_i64(float x) {
    return (x >= -9223372036854775808.0f && x < 9223372036854775808.0f) ? (int64_t)x : INT64_MIN;
}

/* Tensor::to(DType) src/Tensor.cpp:197-243 (from fp32 only) */
int co_cast_from_f32(const float* in, void* out, int dtype, long n) {
    for (long i = 0; i < n; ++i) {
        switch (dtype) {
            case 1: ((double*)out)[i] = (double)in[i]; break;
            case 2: ((int32_t*)out)[i] = f32_to_i32(in[i]); break;
            case 3: ((int64_t*)out)[i] = f32_to_i64(in[i]); break;
            case 4: ((unsigned char*)out)[i] = (unsigned char)(in[i] != 0.0f); break;
            default: return -1;
        }
    }
    return 0;
}

/* The typed arms of Tensor::operator+(float) src/Tensor.cpp:870-890, operator*(float) :766-786
 * and operator/(float) :933-953: the scalar is converted to the tensor's type first (an integer
 * tensor times 2.7f is times 2).  op: 0 '+', 1 '*', 2 '/'.  Integer sums and products wrap (the
 * machine's two's complement arithmetic); -1 for an integer division by a scalar that converts
 * to 0, where the reference's process stops with SIGFPE, as it does for the most negative integer
 * divided by -1, which is stated here as wrapping to itself. */
int co_scalar_op_typed(const void* in, void* out, int dtype, int op, float s, long n) {
    if (op < 0 || op > 2) return -1;
    if (dtype == 1) {
        const double d = (double)s;
        for (long i = 0; i < n; ++i) {
            const double x = ((const double*)in)[i];
            ((double*)out)[i] = op == 0 ? x + d : op == 1 ? x * d : x / d;
        }
    } else if (dtype == 2) {
        const int32_t k = f32_to_i32(s);
        if (op == 2 && k == 0) return -1;
        for (long i = 0; i < n; ++i) {
            const int32_t x = ((const int32_t*)in)[i];
            ((int32_t*)out)[i] = op == 0   ? (int32_t)((uint32_t)x + (uint32_t)k)
                                 : op == 1 ? (int32_t)((uint32_t)x * (uint32_t)k)
                                 : k == -1 ? (int32_t)(0u - (uint32_t)x)
                                           : x / k;
        }
    } else if (dtype == 3) {
        const int64_t k = f32_to_i64(s);
        if (op == 2 && k == 0) return -1;
        for (long i = 0; i < n; ++i) {
            const int64_t x = ((const int64_t*)in)[i];
            ((int64_t*)out)[i] = op == 0   ? (int64_t)((uint64_t)x + (uint64_t)k)
                                 : op == 1 ? (int64_t)((uint64_t)x * (uint64_t)k)
                                 : k == -1 ? (int64_t)((uint64_t)0 - (uint64_t)x)
                                           : x / k;
        }
    } else {
        return -1;
    }
    return 0;
}

/* grad[i] += val[i], the typed arms of src/AutoDiff.cpp:1880-1903 */
int co_accumulate_typed(void* acc, const void* val, int dtype, long n) {
    for (long i = 0; i < n; ++i) {
        switch (dtype) {
            case 1: ((double*)acc)[i] += ((const double*)val)[i]; break;
            case 2: ((int32_t*)acc)[i] = (int32_t)((uint32_t)((int32_t*)acc)[i] + (uint32_t)((const int32_t*)val)[i]); break;
            case 3: ((int64_t*)acc)[i] = (int64_t)((uint64_t)((int64_t*)acc)[i] + (uint64_t)((const int64_t*)val)[i]); break;
            default: return -1;
        }
    }
    return 0;
}

/* Tensor::softmax(dim) for double: src/Tensor.cpp:1686-1696 (1-D: rows = 1, dim = 1), :1749-1764
 * (dim 1), :1765-1781 (dim 0): first maximum, e = exp(x - max) stored, sequential sum, division. */
void co_softmax_f64(const double* x, double* y, long rows, long cols, int dim) {
    const long lines = dim == 1 ? rows : cols, len = dim == 1 ? cols : rows;
    const long step = dim == 1 ? 1 : cols, line_step = dim == 1 ? cols : 1;
    for (long l = 0; l < lines; ++l) {
        const double* in = x + l * line_step;
        double* out = y + l * line_step;
        double m = in[0];
        for (long k = 1; k < len; ++k)
            if (in[k * step] > m) m = in[k * step];
        double sum = 0.0;
        for (long k = 0; k < len; ++k) {
            const double e = exp(in[k * step] - m);
            out[k * step] = e;
            sum += e;
        }
        for (long k = 0; k < len; ++k) out[k * step] /= sum;
    }
}

/* ------------------------------------------------------------- fused expression programs */

/* Extension: the reference evaluates one operator per kernel.  A program is a straight-line list
 * of (op, dst, a, b) over per-element value slots plus one immediate per instruction; each
 * opcode is the per-element body of the function named beside it, so running a program equals
 * calling those functions one after the other on whole tensors.
 *   0 load full input a        1 load row-vector input a (index i % cols)
 *   2 co_add  3 co_sub  4 co_mul  5 co_div  6 co_neg  7 co_relu  8 co_sigmoid  9 co_tanh
 *  10 co_sin  11 co_cos  12 co_scalar_add  13 co_scalar_mul  14 co_scalar_div
 *  15 imm - x (the "1.0f - s" of co_sigmoid_bwd / co_tanh_bwd)   16 co_relu_bwd (a = x, b = g)
 *  17 co_any_abs_lt_eps of slot a into status   18 store slot a to output dst
 *  19 store 0 + slot a (src/AutoDiff.cpp:1870-1907: contributions are added to a zero-filled buffer)
 * Returns 0, or -1 for a malformed program. */
int co_expr_run(const int* prog, const float* imm, int n, const float* const* in, int n_in, float* const* out, int n_out,
                long rows, long cols, int* status) {
    enum { SLOTS = 32 };
    for (int pc = 0; pc < n; ++pc) {
        const int op = prog[4 * pc], d = prog[4 * pc + 1], a = prog[4 * pc + 2], b = prog[4 * pc + 3];
        if (op < 0 || op > 19 || a < 0 || b < 0 || d < 0) return -1;
        if (op <= 1 ? (a >= n_in || d >= SLOTS) : (op >= 18 ? (d >= n_out || a >= SLOTS) : (a >= SLOTS || b >= SLOTS || d >= SLOTS)))
            return -1;
    }
    const long total = rows * cols;
    for (long i = 0; i < total; ++i) {
        float v[SLOTS];
        memset(v, 0, sizeof(v));
        for (int pc = 0; pc < n; ++pc) {
            const int op = prog[4 * pc], d = prog[4 * pc + 1], a = prog[4 * pc + 2], b = prog[4 * pc + 3];
            const float s = imm[pc];
            switch (op) {
                case 0: v[d] = in[a][i]; break;
                case 1: v[d] = in[a][i % cols]; break;
                case 2: v[d] = v[a] + v[b]; break;
                case 3: v[d] = v[a] - v[b]; break;
                case 4: v[d] = v[a] * v[b]; break;
                case 5: v[d] = v[a] / v[b]; break;
                case 6: v[d] = -v[a]; break;
                case 7: v[d] = (0.0f < v[a]) ? v[a] : 0.0f; break;
                case 8: v[d] = 1.0f / (1.0f + expf(-v[a])); break;
                case 9: { float ep = expf(v[a]), en = expf(-v[a]); v[d] = (ep - en) / (ep + en); break; }
                case 10: v[d] = sinf(v[a]); break;
                case 11: v[d] = cosf(v[a]); break;
                case 12: v[d] = v[a] + s; break;
                case 13: v[d] = v[a] * s; break;
                case 14: v[d] = v[a] / s; break;
                case 15: v[d] = s - v[a]; break;
                case 16: { float mask = (v[a] > 0.0f) ? 1.0f : 0.0f; v[d] = v[b] * mask; break; }
                case 17: if (fabsf(v[a]) < FLT_EPSILON && status) *status |= 1; break;
                case 18: out[d][i] = v[a]; break;
                case 19: out[d][i] = 0.0f + v[a]; break;
            }
        }
    }
    return 0;
}

/* ------------------------------------------- gradient shape adjustment, the whole function */

/* src/AutoDiff.cpp:562-1049, check_and_adjust_grad_shape, every branch, for float tensors of up to
 * 8 dimensions.  Returns 0, or -1 where the reference itself reads beyond the end of the gradient
 * (its index arithmetic at :727-757 takes the flat result index as the last coordinate), or -2 for
 * more than 8 dimensions.  gs / ts: shapes, gr / tr: ranks.
 *   :565-567   equal shapes: the gradient itself
 *   :579-627   0-D gradient: every element of the result is its value
 *   :633-687   rank(g) < rank(target): the gradient is copied into a tensor of shape [1, .., 1, g's
 *              dims] element i from element i % numel(g) (the two element counts are equal, so this
 *              is a reshape), then the function calls itself
 *   :690-890   "can broadcast" (every trailing pair of dims equal or one of them 1): result[i] =
 *              0 + g[grad_index(i)]; the coordinate loop :727-732 runs from the LAST dimension with
 *              the full flat index, so the last coordinate is i itself and all others are 0: the
 *              gradient's element i (or element 0 when its last dimension is 1)
 *   :892-966   "can reduce": result[i % numel] += g[i] (unreachable: its condition implies the
 *              previous one; kept in the order of the source)
 *   :968-1046  otherwise: result[i] = sum over j with j % numel(result) == i of g[j], from 0 */
int co_adjust_grad_shape(const float* g, const long* gs, int gr, float* out, const long* ts, int tr) {
    if (gr > 8 || tr > 8) return -2;
    long gn = 1, tn = 1;
    for (int i = 0; i < gr; ++i) gn *= gs[i];
    for (int i = 0; i < tr; ++i) tn *= ts[i];
    int same = gr == tr;
    for (int i = 0; same && i < gr; ++i) same = gs[i] == ts[i];
    if (same) {
        memcpy(out, g, (size_t)gn * sizeof(float));
        return 0;
    }
    if (gr == 0) {
        for (long i = 0; i < tn; ++i) out[i] = g[0];
        return 0;
    }
    if (gr < tr) {
        long ns[8];
        for (int i = 0; i < tr; ++i) ns[i] = 1;
        for (int i = 0; i < gr; ++i) ns[tr - gr + i] = gs[i];
        float* temp = (float*)malloc((size_t)(gn > 0 ? gn : 1) * sizeof(float));
        for (long i = 0; i < gn; ++i) temp[i] = g[i % gn];
        int rc = co_adjust_grad_shape(temp, ns, tr, out, ts, tr);
        free(temp);
        return rc;
    }
    int can_broadcast = 1;
    for (int i = 1; i <= tr; ++i) {
        long gd = gs[gr - i], td = ts[tr - i];
        if (gd != td && gd != 1 && td != 1) { can_broadcast = 0; break; }
    }
    if (can_broadcast) {
        long gstr[8], rstr[8];
        for (int i = gr - 1, a = 1; i >= 0; --i) { gstr[i] = a; a *= gs[i]; }
        for (int i = tr - 1, a = 1; i >= 0; --i) { rstr[i] = a; a *= ts[i]; }
        for (long i = 0; i < tn; ++i) {
            long ri[8] = {0}, gi[8] = {0};
            long temp = i;
            for (int j = tr - 1; j >= 0; --j) {
                ri[j] = temp / rstr[j];
                temp %= rstr[j];
            }
            for (int j = 1; j <= tr; ++j) gi[gr - j] = (gs[gr - j] == 1) ? 0 : ri[tr - j];
            long at = 0;
            for (int j = 0; j < gr; ++j) at += gi[j] * gstr[j];
            if (at >= gn) return -1;
            out[i] = 0.0f + g[at];
        }
        return 0;
    }
    int can_reduce = 1;
    for (int i = 1; i <= (gr < tr ? gr : tr); ++i) {
        long gd = gs[gr - i], td = ts[tr - i];
        if (gd != td && td != 1) { can_reduce = 0; break; }
    }
    if (can_reduce) {
        for (long i = 0; i < tn; ++i) out[i] = 0.0f;
        for (long i = 0; i < gn; ++i) out[i % tn] += g[i];
        return 0;
    }
    for (long i = 0; i < tn; ++i) {
        float sum = 0.0f;
        for (long j = i; j < gn; j += tn) sum += g[j];
        out[i] = sum;
    }
    return 0;
}

/* Extension: the gradient of a broadcast operand as the mathematics has it.  The target shape is
 * padded with leading 1s to the gradient's rank; per dimension the two extents are equal (kept), the
 * target's is 1 (summed over) or the gradient's is 1 (repeated).  Sums in double, in index order.
 * -1: the shapes do not broadcast. */
int co_broadcast_reduce(const float* g, const long* gs, int gr, float* out, const long* ts, int tr) {
    if (gr > 8 || tr > gr) return -1;
    long tp[8], tn = 1;
    for (int i = 0; i < gr; ++i) tp[i] = (i < gr - tr) ? 1 : ts[i - (gr - tr)];
    for (int i = 0; i < gr; ++i) {
        if (tp[i] != gs[i] && tp[i] != 1 && gs[i] != 1) return -1;
        tn *= tp[i];
    }
    long gstr[8];
    for (int i = gr - 1, a = 1; i >= 0; --i) { gstr[i] = a; a *= gs[i]; }
    for (long o = 0; o < tn; ++o) {
        long rem = o, base = 0, red = 1;
        for (int d = gr - 1; d >= 0; --d) {
            long c = rem % tp[d];
            rem /= tp[d];
            if (gs[d] == tp[d]) base += c * gstr[d];
        }
        for (int d = 0; d < gr; ++d) if (tp[d] == 1 && gs[d] > 1) red *= gs[d];
        double sum = 0.0;
        for (long r = 0; r < red; ++r) {
            long q = r, at = base;
            for (int d = gr - 1; d >= 0; --d)
                if (tp[d] == 1 && gs[d] > 1) { at += (q % gs[d]) * gstr[d]; q /= gs[d]; }
            sum += (double)g[at];
        }
        out[o] = (float)sum;
    }
    return 0;
}

/* ------------------- methods the reference declares on Tensor and never defines (extensions) */

/* include/Tensor.h:719 operator-(float), :954-972 abs / exp / log / sqrt, :978 square, :996 tan,
 * :1052 leaky_relu(negative_slope): no bodies exist in the reference, so each is the C++ library call
 * that its name stands for, on floats.  op: 0 abs, 1 exp, 2 log, 3 sqrt, 4 square, 5 tan,
 * 6 leaky_relu (p = slope), 7 a - p. */
void co_unary_ext(int op, const float* a, float p, float* r, long n) {
    for (long i = 0; i < n; ++i) {
        float x = a[i];
        switch (op) {
            case 0: r[i] = fabsf(x); break;
            case 1: r[i] = expf(x); break;
            case 2: r[i] = logf(x); break;
            case 3: r[i] = sqrtf(x); break;
            case 4: r[i] = x * x; break;
            case 5: r[i] = tanf(x); break;
            case 6: r[i] = (x > 0.0f) ? x : x * p; break;
            default: r[i] = x - p; break;
        }
    }
}
/* Their gradients, the factor evaluated in fp32 in the stated order and then multiplied by g:
 * abs sign(x) * g; exp y * g; log g / x; sqrt g / (y * 2); square (x * 2) * g; tan (1 + y * y) * g;
 * leaky_relu g * (x > 0 ? 1 : slope); a - p: g.  v = x for abs, log, square, leaky_relu and the
 * result y for exp, sqrt, tan. */
void co_unary_ext_bwd(int op, const float* v, const float* g, float p, float* dx, long n) {
    for (long i = 0; i < n; ++i) {
        float x = v[i], u = g[i];
        switch (op) {
            case 0: { float s = (x > 0.0f) ? 1.0f : ((x < 0.0f) ? -1.0f : 0.0f); dx[i] = s * u; break; }
            case 1: dx[i] = x * u; break;
            case 2: dx[i] = u / x; break;
            case 3: { float d = x * 2.0f; dx[i] = u / d; break; }
            case 4: { float d = x * 2.0f; dx[i] = d * u; break; }
            case 5: { float yy = x * x; float s = 1.0f + yy; dx[i] = s * u; break; }
            case 6: { float m = (x > 0.0f) ? 1.0f : p; dx[i] = u * m; break; }
            default: dx[i] = u; break;
        }
    }
}

/* include/Tensor.h:824-948: sum / mean / max / min / std / var over a dimension, declared only.
 * x is read as [outer, len, inner]; out[o, i] reduces x[o, :, i].  kind: 0 sum (fp32, in index
 * order, as Tensor::sum() src/Tensor.cpp:644-647 adds), 1 mean (that sum / float(len)), 2 max and
 * 3 min (m = element 0, then `if (v > m)` / `if (v < m)` in index order: the first occurrence wins
 * and a NaN only stays when it comes first; index = its position), 4 var and 5 std (two passes in
 * double: mean, then sum of squared deviations / (len - ddof)); mean_out (4, 5) the mean as a float. */
void co_reduce_dim(int kind, const float* x, float* out, int* index, float* mean_out, long outer, long len, long inner, int ddof) {
    for (long o = 0; o < outer; ++o)
        for (long i = 0; i < inner; ++i) {
            const float* p = x + o * len * inner + i;
            long at = o * inner + i;
            if (kind == 0 || kind == 1) {
                float s = 0.0f;
                for (long l = 0; l < len; ++l) s += p[l * inner];
                out[at] = kind == 0 ? s : s / (float)len;
            } else if (kind == 2 || kind == 3) {
                float m = p[0];
                int pos = 0;
                for (long l = 1; l < len; ++l) {
                    float v = p[l * inner];
                    if (kind == 2 ? (v > m) : (v < m)) { m = v; pos = (int)l; }
                }
                out[at] = m;
                if (index) index[at] = pos;
            } else {
                double mean = 0.0, m2 = 0.0;
                for (long l = 0; l < len; ++l) mean += (double)p[l * inner];
                mean /= (double)len;
                for (long l = 0; l < len; ++l) { double d = (double)p[l * inner] - mean; m2 += d * d; }
                double var = m2 / ((double)len - (double)ddof);
                out[at] = kind == 4 ? (float)var : (float)sqrt(var);
                if (mean_out) mean_out[at] = (float)mean;
            }
        }
}
/* Gradients of the six, every step rounded to fp32 in this order: sum g; mean g / float(len);
 * max / min g at index and +0 elsewhere; var ((x - mean) * 2 / float(len - ddof)) * g;
 * std ((x - mean) / (float(len - ddof) * y)) * g. */
void co_reduce_dim_bwd(int kind, const float* x, const float* y, const int* index, const float* mean, const float* g, float* dx,
                       long outer, long len, long inner, int ddof) {
    for (long o = 0; o < outer; ++o)
        for (long i = 0; i < inner; ++i) {
            long at = o * inner + i;
            float u = g[at];
            float nf = (float)((double)len - (double)ddof);
            for (long l = 0; l < len; ++l) {
                long e = (o * len + l) * inner + i;
                if (kind == 0) dx[e] = u;
                else if (kind == 1) dx[e] = u / (float)len;
                else if (kind == 2 || kind == 3) dx[e] = (l == index[at]) ? u : 0.0f;
                else {
                    float d = x[e] - mean[at];
                    if (kind == 4) { float t = d * 2.0f; float q = t / nf; dx[e] = q * u; }
                    else { float den = nf * y[at]; float q = d / den; dx[e] = q * u; }
                }
            }
        }
}

/* include/Tensor.h:1072 log_softmax(dim), declared only.  In the style of Tensor::softmax
 * (src/Tensor.cpp:1713-1744): m = max (first wins), s = sum of expf(x - m) in index order,
 * y = (x - m) - logf(s).  dim 1: rows, dim 0: columns. */
void co_log_softmax(const float* x, float* y, long rows, long cols, int dim) {
    long runs = dim == 1 ? rows : cols, len = dim == 1 ? cols : rows;
    long step = dim == 1 ? 1 : cols, jump = dim == 1 ? cols : 1;
    for (long r = 0; r < runs; ++r) {
        const float* p = x + r * jump;
        float m = p[0];
        for (long j = 1; j < len; ++j) if (p[j * step] > m) m = p[j * step];
        float s = 0.0f;
        for (long j = 0; j < len; ++j) s += expf(p[j * step] - m);
        float lg = logf(s);
        for (long j = 0; j < len; ++j) { float d = p[j * step] - m; y[r * jump + j * step] = d - lg; }
    }
}
/* its gradient: d = sum of g in index order; dx = g - expf(y) * d */
void co_log_softmax_bwd(const float* y, const float* g, float* dx, long rows, long cols, int dim) {
    long runs = dim == 1 ? rows : cols, len = dim == 1 ? cols : rows;
    long step = dim == 1 ? 1 : cols, jump = dim == 1 ? cols : 1;
    for (long r = 0; r < runs; ++r) {
        float d = 0.0f;
        for (long j = 0; j < len; ++j) d += g[r * jump + j * step];
        for (long j = 0; j < len; ++j) {
            long e = r * jump + j * step;
            float t = expf(y[e]) * d;
            dx[e] = g[e] - t;
        }
    }
}

/* ------------------------------------------------------------------------- input generator */

/* Counter-based generator of this repository (the reference has no seedable one:
 * src/Tensor.cpp:463 seeds from random_device).  z = mix(seed * 0x9E3779B97F4A7C15 + i). */
static uint64_t mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xBF58476D1CE4E5B9ULL;
    z ^= z >> 27;
    z *= 0x94D049BB133111EBULL;
    z ^= z >> 31;
    return z;
}
static uint64_t draw(uint64_t seed, uint64_t i) { return mix64(seed * 0x9E3779B97F4A7C15ULL + i); }

void co_fill_uniform(float* r, long n, uint64_t seed, double lo, double hi) {
    for (long i = 0; i < n; ++i) {
        double u = (double)(draw(seed, (uint64_t)i) >> 40) * (1.0 / 16777216.0);
        r[i] = (float)(lo + (hi - lo) * u);
    }
}
void co_fill_normal(float* r, long n, uint64_t seed, double mean, double sigma) {
    for (long i = 0; i < n; ++i) {
        double u1 = ((double)(draw(seed, (uint64_t)i) >> 11) + 0.5) * (1.0 / 9007199254740992.0);
        double u2 = ((double)(draw(seed ^ 0xA5A5A5A5A5A5A5A5ULL, (uint64_t)i) >> 11) + 0.5) *
                    (1.0 / 9007199254740992.0);
        double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
        r[i] = (float)(mean + sigma * z);
    }
}
void co_fill_int(float* r, long n, uint64_t seed, long range) {
    for (long i = 0; i < n; ++i) r[i] = (float)(draw(seed, (uint64_t)i) % (uint64_t)range);
}
