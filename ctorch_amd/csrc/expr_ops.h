// Per-element building blocks shared by the one-operator kernels, the fused-expression interpreter
// and the fused-expression kernels that are compiled at run time: the lookup tables staged in LDS,
// the reference's tanh and sigmoid formulas on glibc's exponential, and the transcendental
// operators applied to the N elements a lane owns.  This text is also handed to the run-time compiler
// (after devmath.h), so it uses nothing but devmath.h and the device language itself, has no
// includes of its own, and sits at whatever namespace scope includes it.
#ifndef CTAMD_EXPR_OPS_H
#define CTAMD_EXPR_OPS_H

typedef float v4f __attribute__((ext_vector_type(4)));

// Lookup tables of devmath.h staged in LDS once per block (random per-lane indices).
struct Tables {
    const uint64_t* exp2;
    const uint32_t* inv_pio4;
    const double* log;       // cta_log_tab, staged only for functors with kLogTable
};

// num / den for the tanh quotient below (den >= 2, |num| <= den): the steps of the division the compiler
// writes for `/` - reciprocal, one Newton step on it, the quotient, two corrections on exact residuals -
// without that sequence's operand scaling and fix-up instructions, which take as long as the
// rest together and only matter for operands this quotient does not have.  den >= 2^100 (|x| > 69),
// infinite (inf / inf = NaN for |x| > 88.72) or NaN takes the plain division.  The same bits as `/`:
// every float through the tanh kernel against the quotient formed by the division kernel
// (tests/test_gpu_parity.py, all 2^32 arguments).
__device__ __forceinline__ float tanh_quotient(float num, float den) {
    float y = __builtin_amdgcn_rcpf(den);
    y = __fmaf_rn(__fmaf_rn(-den, y, 1.0f), y, y);
    float q = num * y;
    q = __fmaf_rn(__fmaf_rn(-den, q, num), y, q);
    q = __fmaf_rn(__fmaf_rn(-den, q, num), y, q);
    if (__builtin_expect(!(den < 0x1p100f), 0)) q = num / den;
    return q;
}
__device__ __forceinline__ float tanh_ref(float x, const Tables& t) {
    float ep, en;
    cta_expf_pair(x, t.exp2, &ep, &en);
    return tanh_quotient(ep - en, ep + en);
}
__device__ __forceinline__ float sigmoid_ref(float x, const Tables& t) {
    return 1.0f / (1.0f + cta_expf_tab(-x, t.exp2));
}
__device__ __forceinline__ void stage_tables(uint64_t* exp2, uint32_t* pio4) {
    if (threadIdx.x < 32) exp2[threadIdx.x] = cta_exp2_tab[threadIdx.x];
    if (threadIdx.x >= 32 && threadIdx.x < 56) pio4[threadIdx.x - 32] = cta_inv_pio4[threadIdx.x - 32];
    __syncthreads();
}


// One operator on the N elements of a lane, in place: c holds operand a on entry and the result on
// return, b the second operand of the two-operand operators.  The operator is chosen once (a
// scalar branch) and its N evaluations are independent instruction streams that the compiler
// interleaves: the long dependent chains of the transcendental functors hide each other's latencies.
template <int N, class F>
__device__ __forceinline__ void each(float (&c)[N], F f) {
#pragma unroll
    for (int e = 0; e < N; ++e) c[e] = f(e);
}
// FASTM: sin, cos and sigmoid in single precision (sin / cos within 2 ulp of sinf / cosf for |x| < 120,
// sigmoid within 2 ulp of the reference's formula on expf for -16.625 <= x <= 128; the
// double-precision routines beyond); otherwise the routines that return glibc's floats.
template <bool FASTM, int WANT_COS, int N>
__device__ __forceinline__ void sin_or_cos(float (&c)[N], const Tables& t) {
    bool rare = false;
    float x[N];
#pragma unroll
    for (int e = 0; e < N; ++e) {
        x[e] = c[e];
        c[e] = FASTM ? cta_sincosf_f32(x[e], WANT_COS) : cta_sincosf_fast(x[e], WANT_COS);
        rare = rare || !(__builtin_fabsf(x[e]) < 120.0f);      // |x| >= 120, inf, NaN
    }
    if (__builtin_expect(rare, 0)) {
        for (int e = 0; e < N; ++e)
            if (cta_sincos_is_rare(x[e])) c[e] = cta_sincosf(x[e], WANT_COS, t.inv_pio4);
    }
}

// Sigmoid in single precision (within 2 ulp of the reference's formula on expf) for -16.625 <= x <= 128;
// a wave with an element outside that, or a NaN, repairs those elements with the double-precision routine.
template <int N>
__device__ __forceinline__ void sigmoid_fast(float (&c)[N], const Tables& t) {
    bool rare = false;
    float x[N];
#pragma unroll
    for (int e = 0; e < N; ++e) {
        x[e] = c[e];
        c[e] = cta_sigmoid_f32(x[e]);
        rare = rare || cta_sigmoid_is_rare(x[e]);
    }
    if (__builtin_expect(rare, 0)) {
        for (int e = 0; e < N; ++e)
            if (cta_sigmoid_is_rare(x[e])) c[e] = sigmoid_ref(x[e], t);
    }
}

#endif
