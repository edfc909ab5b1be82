// Per-element functors of the elementwise kernels: the reference's fp32 operation order for every
// forward operator and for the tape's gradient arithmetic.  Shared by the one-operator kernels
// (elementwise.hip) and the fused-expression interpreter (expr.hip).  Files that include this must
// be compiled with -ffp-contract=off: a fused multiply-add would change the bits.
#ifndef CTAMD_FUNCTORS_H
#define CTAMD_FUNCTORS_H

#include "common.h"
#include "devmath.h"

namespace ctamd {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

#include "expr_ops.h"

template <int N>
struct Ptrs {
    const float* p[N > 0 ? N : 1];
};

// ------------------------------------------------------------------------------- functors
// Each functor: kIn inputs, kTables whether it needs the LDS tables, and
// float operator()(const float* x, const Tables&) with x[0..kIn).

struct AddF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return x[0] + x[1]; } };
struct SubF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return x[0] - x[1]; } };
struct MulF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return x[0] * x[1]; } };
struct DivF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return x[0] / x[1]; } };

// a (op) s with s held in the functor (host scalar) - Tensor::operator+(float) etc.
template <class Op>
struct ScalarF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    float s;
    __device__ float operator()(const float* x, const Tables& t) const { float v[2] = {x[0], s}; return Op()(v, t); } };
// a (op) *s with s a one-element device tensor
template <class Op>
struct DevScalarF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    const float* s;
    __device__ float operator()(const float* x, const Tables& t) const { float v[2] = {x[0], *s}; return Op()(v, t); } };
// *s - b
struct RSubDevScalarF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    const float* s;
    __device__ float operator()(const float* x, const Tables&) const { return *s - x[0]; } };

// a / s for one divisor shared by all elements: the correctly rounded quotient through the
// divisor's double-precision reciprocal (devmath.h, cta_div_rcp) - 3 instructions instead of the
// ~12 of a full fp32 division.
struct DivByRcpF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    double rcp;
    __device__ float operator()(const float* x, const Tables&) const { return cta_div_rcp(x[0], rcp); } };

struct NegF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return -x[0]; } };
// std::max(0.0f, x): (0 < x) ? x : +0  (NaN and -0 give +0)
struct ReluF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return (0.0f < x[0]) ? x[0] : 0.0f; } };
// Sin / Cos family: `operator()` is the straight-line path for |x| < 120; `rare(x)` tells when an
// element needs `slow()` (the table-driven reduction for huge arguments, inf, NaN).  The kernel
// runs the fast path for every element and repairs the rare ones afterwards, so the common case
// carries no per-element branch.
struct SinF { static constexpr int kIn = 1; static constexpr bool kTables = true; static constexpr bool kRare = true;
    __device__ float operator()(const float* x, const Tables&) const { return cta_sincosf_fast(x[0], 0); }
    __device__ bool rare(const float* x) const { return cta_sincos_is_rare(x[0]); }
    __device__ float slow(const float* x, const Tables& t) const { return cta_sincosf(x[0], 0, t.inv_pio4); } };
struct CosF { static constexpr int kIn = 1; static constexpr bool kTables = true; static constexpr bool kRare = true;
    __device__ float operator()(const float* x, const Tables&) const { return cta_sincosf_fast(x[0], 1); }
    __device__ bool rare(const float* x) const { return cta_sincos_is_rare(x[0]); }
    __device__ float slow(const float* x, const Tables& t) const { return cta_sincosf(x[0], 1, t.inv_pio4); } };

struct TanhF { static constexpr int kIn = 1; static constexpr bool kTables = true;
    __device__ float operator()(const float* x, const Tables& t) const { return tanh_ref(x[0], t); } };
struct SigmoidF { static constexpr int kIn = 1; static constexpr bool kTables = true;
    __device__ float operator()(const float* x, const Tables& t) const { return sigmoid_ref(x[0], t); } };

// ---- the operators the reference declares without defining (include/Tensor.h:954-996, :1052); the
// semantics are the C++ library calls their names stand for: std::fabs, std::exp, std::log,
// std::sqrt, x * x, std::tan on floats, and leaky ReLU as x > 0 ? x : x * slope
struct AbsF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return __builtin_fabsf(x[0]); } };
struct ExpF { static constexpr int kIn = 1; static constexpr bool kTables = true;
    __device__ float operator()(const float* x, const Tables& t) const { return cta_expf_tab(x[0], t.exp2); } };
struct LogF { static constexpr int kIn = 1; static constexpr bool kTables = false; static constexpr bool kLogTable = true;
    __device__ float operator()(const float* x, const Tables& t) const { return cta_logf(x[0], t.log); } };
struct SqrtF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return __builtin_sqrtf(x[0]); } };   // IEEE, correctly rounded (the build keeps fp32 sqrt and divide correctly rounded)
struct SquareF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const { return x[0] * x[0]; } };
struct TanF { static constexpr int kIn = 1; static constexpr bool kTables = true; static constexpr bool kRare = true;
    __device__ float operator()(const float* x, const Tables&) const { return cta_tanf_fast(x[0]); }
    __device__ bool rare(const float* x) const { return cta_sincos_is_rare(x[0]); }
    __device__ float slow(const float* x, const Tables& t) const { return cta_tanf(x[0], t.inv_pio4); } };
struct LeakyReluF { static constexpr int kIn = 1; static constexpr bool kTables = false;
    float slope;
    __device__ float operator()(const float* x, const Tables&) const { return (x[0] > 0.0f) ? x[0] : x[0] * slope; } };

// ---- their gradients; inputs (x or y, g).  Exp's is y * g and Log's g / x: the Mul and Div kernels.
struct AbsBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;     // sign(x) * g
    __device__ float operator()(const float* x, const Tables&) const {
        float s = (x[0] > 0.0f) ? 1.0f : ((x[0] < 0.0f) ? -1.0f : 0.0f);
        return s * x[1]; } };
struct SqrtBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;    // g / (y * 2)
    __device__ float operator()(const float* x, const Tables&) const {
        float d = x[0] * 2.0f;
        return x[1] / d; } };
struct SquareBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;  // (x * 2) * g
    __device__ float operator()(const float* x, const Tables&) const {
        float d = x[0] * 2.0f;
        return d * x[1]; } };
struct TanBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;     // (1 + y * y) * g
    __device__ float operator()(const float* x, const Tables&) const {
        float yy = x[0] * x[0];
        float s = 1.0f + yy;
        return s * x[1]; } };
struct LeakyReluBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;   // g * (x > 0 ? 1 : slope)
    float slope;
    __device__ float operator()(const float* x, const Tables&) const {
        float m = (x[0] > 0.0f) ? 1.0f : slope;
        return x[1] * m; } };

// ---- gradient arithmetic; inputs (x, g) unless noted
struct ReluBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const {
        float mask = (x[0] > 0.0f) ? 1.0f : 0.0f;
        return x[1] * mask; } };
struct SigmoidBwdF { static constexpr int kIn = 2; static constexpr bool kTables = true;
    __device__ float operator()(const float* x, const Tables& t) const {
        float s = sigmoid_ref(x[0], t);
        float om = 1.0f - s;
        float p = s * om;
        return p * x[1]; } };
struct TanhBwdF { static constexpr int kIn = 2; static constexpr bool kTables = true;
    __device__ float operator()(const float* x, const Tables& t) const {
        float th = tanh_ref(x[0], t);
        float tt = th * th;
        float om = 1.0f - tt;
        return om * x[1]; } };
struct SinBwdF { static constexpr int kIn = 2; static constexpr bool kTables = true; static constexpr bool kRare = true;
    __device__ float operator()(const float* x, const Tables&) const { return cta_sincosf_fast(x[0], 1) * x[1]; }
    __device__ bool rare(const float* x) const { return cta_sincos_is_rare(x[0]); }
    __device__ float slow(const float* x, const Tables& t) const { return cta_sincosf(x[0], 1, t.inv_pio4) * x[1]; } };
struct CosBwdF { static constexpr int kIn = 2; static constexpr bool kTables = true; static constexpr bool kRare = true;
    __device__ float operator()(const float* x, const Tables&) const { return (-cta_sincosf_fast(x[0], 0)) * x[1]; }
    __device__ bool rare(const float* x) const { return cta_sincos_is_rare(x[0]); }
    __device__ float slow(const float* x, const Tables& t) const { return (-cta_sincosf(x[0], 0, t.inv_pio4)) * x[1]; } };
// inputs (p, t); rfn = 1.0 / double(float(n)); g a 0-D device tensor
struct MseBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    double rfn; const float* g;
    __device__ float operator()(const float* x, const Tables&) const {
        float d = x[0] - x[1];
        float d2 = d * 2.0f;
        float q = cta_div_rcp(d2, rfn);          // d2 / float(n)
        return 0.0f + q * *g; } };   // "0 +": the tape adds the term to a zero-filled buffer (-0 becomes +0)
struct MaeBwdF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    double rfn; const float* g;
    __device__ float operator()(const float* x, const Tables&) const {
        float d = x[0] - x[1];
        float s = (d > 0.0f) ? 1.0f : ((d < 0.0f) ? -1.0f : 0.0f);
        float q = cta_div_rcp(s, rfn);           // sign / float(n)
        return 0.0f + q * *g; } };   // "0 +": the tape adds the term to a zero-filled buffer (-0 becomes +0)
// inputs (F's inputs..., acc): acc + F(...) - a gradient term added to the gradient gathered so far in
// the pass that forms it (the term is rounded before the addition, as the separate accumulate pass adds it)
template <class F>
struct PlusF { static constexpr int kIn = F::kIn + 1; static constexpr bool kTables = F::kTables;
    F f;
    __device__ float operator()(const float* x, const Tables& t) const {
        float term = f(x, t);
        return x[F::kIn] + term; } };
// the same around a functor with a rare slow path (SinBwdF, CosBwdF)
template <class F>
struct PlusRareF : PlusF<F> { static constexpr bool kRare = true;
    __device__ bool rare(const float* x) const { return this->f.rare(x); }
    __device__ float slow(const float* x, const Tables& t) const {
        float term = this->f.slow(x, t);
        return x[F::kIn] + term; } };
// inputs (a, b, g): ((-a) * g) / (b * b)
struct DivBwdBF { static constexpr int kIn = 3; static constexpr bool kTables = false;
    __device__ float operator()(const float* x, const Tables&) const {
        float na = -x[0];
        float num = na * x[2];
        float den = x[1] * x[1];
        return num / den; } };
// optimiser update p - g * lr with the product rounded first (mnist/mnist.cpp:86-92; that file is
// built without FMA contraction by the reference); inputs (p, g)
struct SgdF { static constexpr int kIn = 2; static constexpr bool kTables = false;
    float lr;
    __device__ float operator()(const float* x, const Tables&) const {
        float step = x[1] * lr;
        return x[0] - step; } };
struct FillF { static constexpr int kIn = 0; static constexpr bool kTables = false;
    float v;
    __device__ float operator()(const float*, const Tables&) const { return v; } };
struct FillFromF { static constexpr int kIn = 0; static constexpr bool kTables = false;
    const float* v;
    __device__ float operator()(const float*, const Tables&) const { return *v; } };

__device__ __forceinline__ void stage_log_table(double* tab) {
    if (threadIdx.x < 32) tab[threadIdx.x] = cta_log_tab[threadIdx.x];
    __syncthreads();
}
}  // namespace
}  // namespace ctamd

#endif
