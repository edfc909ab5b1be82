// Transcendentals of the device kernels: expf, logf, sinf, cosf evaluated in fp64 and rounded to
// fp32 once.
//
// The reference's CPU kernels call glibc's float routines (Sin_/Cos_/Tanh_/Sigmoid_/Softmax_/
// CrossEntropy_BASIC_kernel.cpp), and its tanh is (e^x - e^-x)/(e^x + e^-x) in fp32, which
// amplifies a one-ulp difference in expf into hundreds of ulps near zero.  Matching that formula
// therefore needs an expf that returns the same float as glibc's for (nearly) every input, not
// merely an accurate one.  glibc >= 2.27 computes expf/sinf/cosf in double precision with the
// published algorithms of ARM's optimized-routines (2^(k/32) table + cubic for expf; quadrant
// reduction + two short polynomials for sinf/cosf).  The functions below follow those published
// algorithms with the same constants.  Which double operations are fused matters for about one
// input in 10^9; the fused multiply-adds are spelled out below (CTA_FMA) in the places where
// glibc's x86-64 FMA build has them, and every file that includes this header is compiled with
// -ffp-contract=off.  With that, tests/native/devmath_check.c finds zero mismatches against
// glibc 2.35 over all 2^32 floats for expf and over every |x| < 120 for sinf / cosf on the host,
// where this header compiles unchanged; fp64 add / mul / fma are IEEE on CDNA, so the device
// returns the same bits.
//
// Everything here is plain C99-compatible so that the same text is compiled by hipcc for the
// device and by gcc for that host check.
#ifndef CTORCH_AMD_DEVMATH_H
#define CTORCH_AMD_DEVMATH_H

#include <stdint.h>

#if defined(__HIPCC__)
#define CTA_FN __device__ __forceinline__ static
#define CTA_TAB_SPACE __device__ static const
#define CTA_FMA(a, b, c) __fma_rn((a), (b), (c))
#define CTA_FMAF(a, b, c) __fmaf_rn((a), (b), (c))
#else
#define CTA_FMA(a, b, c) __builtin_fma((a), (b), (c))
#define CTA_FMAF(a, b, c) __builtin_fmaf((a), (b), (c))
#include <math.h>
#include <string.h>
#define CTA_FN static inline
#define CTA_TAB_SPACE static const
#endif

CTA_FN uint32_t cta_f2u(float f) {
#if defined(__HIPCC__)
    return __float_as_uint(f);
#else
    uint32_t u; memcpy(&u, &f, 4); return u;
#endif
}
CTA_FN float cta_u2f(uint32_t u) {
#if defined(__HIPCC__)
    return __uint_as_float(u);
#else
    float f; memcpy(&f, &u, 4); return f;
#endif
}
CTA_FN uint64_t cta_d2u(double d) {
#if defined(__HIPCC__)
    return (uint64_t)__double_as_longlong(d);
#else
    uint64_t u; memcpy(&u, &d, 8); return u;
#endif
}
CTA_FN double cta_u2d(uint64_t u) {
#if defined(__HIPCC__)
    return __longlong_as_double((long long)u);
#else
    double d; memcpy(&d, &u, 8); return d;
#endif
}

// a / b for a divisor shared by many elements: with rcp_b = 1.0 / (double)b computed once,
// the double product q = (double)a * rcp_b lies within 2^-52 (relative) of the exact quotient.
// Normal results: the exact quotient of two 24-bit significands is at least 2^-49 (relative) away
// from every midpoint between adjacent floats and can never sit on one (that would need 2^25 to
// divide a 24-bit integer), so (float)q is the correctly rounded fp32 quotient.  Subnormal results
// are rounded at a fixed position (multiples of 2^-149), where the exact quotient CAN be a midpoint
// (a = 147 * 2^-149, b = 98) and q, a hair off it, would break the tie the wrong way.  There, in
// units of 2^-150, a quotient that is not an integer is at least 2^-24 away from every integer while
// q is at most 2^-28 away from the quotient: a q within 2^-26 of an integer is moved onto it, which
// restores every exact quotient - the midpoints among them - and touches nothing else.  Zeros,
// infinities and NaN come out as IEEE division gives them.  tests/native/divcheck.c compares it with
// `a / b` on random pairs and on the midpoint family a = M * B * 2^-149, b = 2 * B.
CTA_FN float cta_div_rcp(float a, double rcp_b) {
    double q = (double)a * rcp_b;
    if (__builtin_expect(__builtin_fabs(q) < 0x1p-126, 0)) {
        double t = q * 0x1p150;
        double m = __builtin_rint(t);
        if (__builtin_fabs(t - m) < 0x1p-26) q = m * 0x1p-150;
    }
    return (float)q;
}

// tab[i] = bits(2^(i/32)) - (i << 47): adding k << 47 yields bits(2^(k/32)) for any integer k.
CTA_TAB_SPACE uint64_t cta_exp2_tab[32] = {
    0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
    0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
    0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
    0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
    0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
    0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
    0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
    0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL};

// `tab` is where the caller keeps the 32 entries (LDS on the device, the array above on the host).
// Valid for every float: NaN -> NaN, +inf -> +inf, -inf -> 0, overflow -> +inf, underflow ->
// correctly rounded subnormals and then 0.  Branch-free: |x| is clamped to 128 first (NaN passes
// through), where the double-precision result is still finite and its conversion to float
// overflows to +inf / rounds to 0 exactly where glibc's range checks return those values.
CTA_FN float cta_exp_clamp(float x) {
    uint32_t ux = cta_f2u(x);
    float ax = cta_u2f(ux & 0x7fffffffu);
    return (ax > 128.0f) ? cta_u2f((ux & 0x80000000u) | 0x43000000u) : x;
}
CTA_FN float cta_expf_tab(float x, const uint64_t* tab) {
    double xd = (double)cta_exp_clamp(x);
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    double kd = CTA_FMA(inv_ln2_n, xd, 0x1.8p+52);   // round to nearest integer in the low bits
    uint64_t ki = cta_d2u(kd);
    kd -= 0x1.8p+52;
    double r = CTA_FMA(inv_ln2_n, xd, -kd);
    uint64_t t = tab[ki & 31u] + (ki << 47);
    double s = cta_u2d(t);
    double p = CTA_FMA(0x1.c6af84b912394p-5 / 32768.0, r, 0x1.ebfce50fac4f3p-3 / 1024.0);
    double r2 = r * r;
    double y = CTA_FMA(0x1.62e42ff0c52d6p-1 / 32.0, r, 1.0);
    y = CTA_FMA(p, r2, y);
    y = y * s;
    return (float)y;
}

// The same for arguments known to be <= 0 or NaN (x - max(x) in softmax): only the lower clamp.
CTA_FN float cta_expf_nonpos(float x, const uint64_t* tab) {
    float xc = (x < -128.0f) ? -128.0f : x;        // NaN stays NaN
    double xd = (double)xc;
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    double kd = CTA_FMA(inv_ln2_n, xd, 0x1.8p+52);
    uint64_t ki = cta_d2u(kd);
    kd -= 0x1.8p+52;
    double r = CTA_FMA(inv_ln2_n, xd, -kd);
    double s = cta_u2d(tab[ki & 31u] + (ki << 47));
    double p = CTA_FMA(0x1.c6af84b912394p-5 / 32768.0, r, 0x1.ebfce50fac4f3p-3 / 1024.0);
    double r2 = r * r;
    double y = CTA_FMA(0x1.62e42ff0c52d6p-1 / 32.0, r, 1.0);
    y = CTA_FMA(p, r2, y);
    return (float)(y * s);
}

// exp(x) and exp(-x) together (tanh needs both).  The reduction of -x is the mirror image of the
// reduction of x - round-to-nearest-even is symmetric, so k' = -k and r' = -r exactly - hence
// only the table entry and the polynomial are evaluated twice.
CTA_FN void cta_expf_pair(float x, const uint64_t* tab, float* e_pos, float* e_neg) {
    double xd = (double)cta_exp_clamp(x);
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    const double c0 = 0x1.c6af84b912394p-5 / 32768.0, c1 = 0x1.ebfce50fac4f3p-3 / 1024.0,
                 c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    double kd = CTA_FMA(inv_ln2_n, xd, 0x1.8p+52);
    uint64_t ki = cta_d2u(kd);
    kd -= 0x1.8p+52;
    double r = CTA_FMA(inv_ln2_n, xd, -kd);
    double r2 = r * r;
    uint64_t nki = 0u - ki;                       // low bits and the shifted-in exponent of -k
    double s_pos = cta_u2d(tab[ki & 31u] + (ki << 47));
    double s_neg = cta_u2d(tab[nki & 31u] + (nki << 47));
    double y_pos = CTA_FMA(CTA_FMA(c0, r, c1), r2, CTA_FMA(c2, r, 1.0)) * s_pos;
    double y_neg = CTA_FMA(CTA_FMA(-c0, r, c1), r2, CTA_FMA(-c2, r, 1.0)) * s_neg;
    *e_pos = (float)y_pos;
    *e_neg = (float)y_neg;
}

// sin / cos: |x| < 0.75 direct, |x| < 120 quadrant reduction with one multiply by pi/2 in double
// (exact enough: 53-bit pi/2 times |n| < 2^7), beyond that `big` reduces x (any accurate fp64
// routine; the caller passes the platform's).  sel = 0 sine, 1 cosine.
CTA_FN double cta_sin_poly(double x, double x2) {
    double x3 = x * x2;
    double s1 = CTA_FMA(x2, -0x1.994eb3774cf24p-13, 0x1.1107605230bc4p-7);
    double x7 = x3 * x2;
    double s = CTA_FMA(x3, -0x1.555545995a603p-3, x);
    return CTA_FMA(x7, s1, s);
}
CTA_FN double cta_cos_poly(double x2) {
    double x4 = x2 * x2;
    double c2 = CTA_FMA(x2, 0x1.99343027bf8c3p-16, -0x1.6c087e89a359dp-10);
    double c1 = CTA_FMA(x2, -0x1.ffffffd0c621cp-2, 0x1p0);
    double x6 = x4 * x2;
    double c = CTA_FMA(x4, 0x1.55553e1068f19p-5, c1);
    return CTA_FMA(x6, c2, c);
}

// 32-bit windows of the binary expansion of 2/pi, each shifted 8 bits from the previous one.
CTA_TAB_SPACE uint32_t cta_inv_pio4[24] = {
    0x000000a2u, 0x0000a2f9u, 0x00a2f983u, 0xa2f9836eu, 0xf9836e4eu, 0x836e4e44u,
    0x6e4e4415u, 0x4e441529u, 0x441529fcu, 0x1529fc27u, 0x29fc2757u, 0xfc2757d1u,
    0x2757d1f5u, 0x57d1f534u, 0xd1f534ddu, 0xf534ddc0u, 0x34ddc0dbu, 0xddc0db62u,
    0xc0db6295u, 0xdb629599u, 0x6295993cu, 0x95993c43u, 0x993c4390u, 0x3c439041u};

// |x| >= 120: multiply the 24-bit significand by 96 bits of 2/pi chosen by the exponent; the top
// two bits of the 64-bit product fraction are the quadrant, the rest the reduced argument.
CTA_FN double cta_reduce_large(uint32_t xi, int* np, const uint32_t* inv_pio4) {
    const uint32_t* arr = inv_pio4 + ((xi >> 26) & 15);
    int shift = (int)((xi >> 23) & 7);
    xi = (xi & 0xffffffu) | 0x800000u;
    xi <<= shift;
    uint64_t res0 = (uint64_t)(uint32_t)(xi * arr[0]);
    uint64_t res1 = (uint64_t)xi * arr[4];
    uint64_t res2 = (uint64_t)xi * arr[8];
    res0 = (res2 >> 32) | (res0 << 32);
    res0 += res1;
    uint64_t n = (res0 + (1ULL << 61)) >> 62;
    res0 -= n << 62;
    double x = (double)(int64_t)res0;
    *np = (int)n;
    return x * 0x1.921FB54442D18p-62;
}

// sinf (want_cos = 0) / cosf (want_cos = 1) for every float.  One straight-line path serves
// |y| < 120: for |y| < 0.75 the quadrant is 0 and the reduced argument is y itself, so glibc's
// separate small-argument branches give the same bits (checked over all floats); beyond 120 the
// 2/pi table reduction runs instead, and inf / NaN give NaN.  The quadrant's sign is applied to the
// rounded float (both polynomials are odd / even in a way that commutes with rounding).
CTA_FN float cta_sincos_finish(float y, uint32_t ay, int want_cos, int n, double xr) {
    if (want_cos) n += 1;                          // cos(x) = sin(x + pi/2)
    double x2 = xr * xr;
    double c = cta_cos_poly(x2);
    double sn = cta_sin_poly(xr, x2);
    double res = (n & 1) ? c : sn;                 // both evaluated: lanes of a wave differ anyway
    float f = cta_u2f(cta_f2u((float)res) ^ ((uint32_t)(n & 2) << 30));
    if (!want_cos) f = (ay < 0x39800000u) ? y : f;   // |y| < 2^-12: sin(y) = y, keeps the sign of -0
    return f;
}
// Straight-line path, correct for |y| < 120 (cta_sincos_is_rare(y) == 0).
CTA_FN float cta_sincosf_fast(float y, int want_cos) {
    uint32_t ay = cta_f2u(y) & 0x7fffffffu;
    double x = (double)y;
    double r = x * 0x1.45F306DC9C883p+23;          // 2/pi scaled by 2^24
    int n = ((int32_t)r + 0x800000) >> 24;         // nearest quadrant
    double xr = CTA_FMA(-(double)n, 0x1.921FB54442D18p0, x);
    return cta_sincos_finish(y, ay, want_cos, n, xr);
}
CTA_FN int cta_sincos_is_rare(float y) { return (cta_f2u(y) & 0x7fffffffu) >= 0x42f00000u; }
// Every float (the |y| >= 120, inf and NaN cases included).
CTA_FN float cta_sincosf(float y, int want_cos, const uint32_t* inv_pio4) {
    if (!cta_sincos_is_rare(y)) return cta_sincosf_fast(y, want_cos);
    uint32_t uy = cta_f2u(y);
    uint32_t ay = uy & 0x7fffffffu;
    if (ay >= 0x7f800000u) return y - y;           // inf, NaN -> NaN
    int n;
    double xr = cta_reduce_large(uy, &n, inv_pio4);
    if (!want_cos) n += (int)(uy >> 31) * 2;       // reduced |y|; sin is odd: sin(t + pi) = -sin(t)
    return cta_sincos_finish(y, ay, want_cos, n, xr);
}

// logf: glibc's algorithm (the published ARM optimized-routines logf: x = 2^k * z with z in
// [0x1.66p-1, 0x1.66p0), 16 subintervals with tabulated 1/c and log(c), a cubic in r = z/c - 1, all
// in double) with the same constants.  cta_log_tab[2*i] = 1/c_i, [2*i+1] = log(c_i).  Returns
// glibc 2.35's float for every input (checked over all 2^32 bit patterns by
// tests/native/devmath_check.c): log(+-0) = -inf, log(x < 0) = NaN, log(inf) = inf, subnormals exact.
CTA_TAB_SPACE double cta_log_tab[32] = {
    0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2, 0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2,
    0x1.49539f0f010bp+0,  -0x1.01eae7f513a67p-2, 0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3,
    0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3, 0x1.25e227b0b8eap+0,  -0x1.1aa2bc79c81p-3,
    0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4, 0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4,
    0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5, 0x1p+0,               0x0p+0,
    0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5,  0x1.ca4b31f026aap-1,  0x1.c5e53aa362eb4p-4,
    0x1.b2036576afce6p-1, 0x1.526e57720db08p-3,  0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3,
    0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2,  0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2};
// `tab`: where the caller keeps the 32 doubles (LDS on the device, the array above on the host).
CTA_FN float cta_logf(float x, const double* tab) {
    uint32_t ix = cta_f2u(x);
    uint32_t special = 0;                      // 1: -inf, 2: x itself (+inf), 3: NaN
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
        if (ix * 2u == 0u) special = 1;
        else if (ix == 0x7f800000u) special = 2;
        else if ((ix & 0x80000000u) || ix * 2u >= 0xff000000u) special = 3;
        else ix = cta_f2u(x * 0x1p23f) - (23u << 23);      // subnormal: normalise
    }
    uint32_t tmp = ix - 0x3f330000u;
    uint32_t i = (tmp >> 19) & 15u;
    int32_t k = (int32_t)tmp >> 23;
    uint32_t iz = ix - (tmp & 0xff800000u);
    double invc = tab[2 * i], logc = tab[2 * i + 1];
    double z = (double)cta_u2f(iz);
    double r = CTA_FMA(z, invc, -1.0);
    double y0 = CTA_FMA((double)k, 0x1.62e42fefa39efp-1, logc);
    double r2 = r * r;
    double y = CTA_FMA(0x1.5575b0be00b6ap-2, r, -0x1.ffffef20a4123p-2);
    y = CTA_FMA(-0x1.00ea348b88334p-2, r2, y);
    y = CTA_FMA(y, r2, y0 + r);
    float f = (float)y;
    if (special == 1) f = -__builtin_huge_valf();
    if (special == 2) f = x;
    if (special == 3) f = x - x, f = (f != f) ? f : __builtin_nanf("");     // NaN (x - x is 0 for finite negatives)
    return f;
}

// tanf as the quotient of the sine and cosine polynomials of one reduced argument, in double,
// rounded once: within 1 ulp of the correctly rounded tangent and of glibc 2.35's tanf (an fdlibm
// routine in float arithmetic that this does not restate) over all floats
// (tests/native/devmath_check.c).  tan(+-0) = +-0, inf / NaN -> NaN.
CTA_FN float cta_tan_finish(float y, uint32_t ay, int n, double xr) {
    double x2 = xr * xr;
    double c = cta_cos_poly(x2);
    double sn = cta_sin_poly(xr, x2);
    // tan = sin / cos in even quadrants, -cos / sin in odd ones.  The quotient through a reciprocal
    // refined once in double from a single-precision start (relative error ~1e-14, far below the
    // polynomials' own): a double-precision division costs more than the rest of the function.
    double num = (n & 1) ? -c : sn;
    double den = (n & 1) ? sn : c;
#if defined(__HIPCC__)
    double r0 = (double)__builtin_amdgcn_rcpf((float)den);
#else
    double r0 = (double)(1.0f / (float)den);
#endif
    double e = CTA_FMA(-den, r0, 1.0);
    double r1 = CTA_FMA(r0, e, r0);
    float f = (float)(num * r1);
    return (ay < 0x39000000u) ? y : f;             // |y| < 2^-13: tan(y) = y, keeps the sign of -0
}
// Straight-line path, correct for |y| < 120 (cta_sincos_is_rare(y) == 0).
CTA_FN float cta_tanf_fast(float y) {
    uint32_t ay = cta_f2u(y) & 0x7fffffffu;
    double x = (double)y;
    double r = x * 0x1.45F306DC9C883p+23;
    int n = ((int32_t)r + 0x800000) >> 24;
    double xr = CTA_FMA(-(double)n, 0x1.921FB54442D18p0, x);
    return cta_tan_finish(y, ay, n, xr);
}
CTA_FN float cta_tanf(float y, const uint32_t* inv_pio4) {
    if (!cta_sincos_is_rare(y)) return cta_tanf_fast(y);
    uint32_t uy = cta_f2u(y);
    uint32_t ay = uy & 0x7fffffffu;
    if (ay >= 0x7f800000u) return y - y;
    int n;
    double xr = cta_reduce_large(uy, &n, inv_pio4);     // reduces |y|; tan is odd
    if (uy >> 31) { xr = -xr; n = -n; }
    return cta_tan_finish(y, ay, n, xr);
}

// ----------------------------------------------------------------------------------------------
// Single-precision sine / cosine for |y| < 120 (cta_sincos_is_rare(y) == 0), for the kernels whose
// time the double-precision routines above would set (fused expressions).  y = k pi/2 + r with k the
// nearest integer and |r| <= pi/4 (1 + 1e-4); sin r from an odd polynomial of degree 7, cos r from
// an even one of degree 8 (fitted on that interval to 4e-9 and 6e-11 relative), and the quadrant
// k mod 4 picks which of the two, and with which sign, is the sine and which the cosine.  pi/2 is
// split in three floats whose first two have 17 significant bits, so the first step of the
// reduction is exact (|k| < 2^7) and the second loses half an ulp of r at most.  Everything up to
// the pick is the same for the sine and the cosine of one argument: a kernel that needs both (a
// product's gradient, sin and cos of one tensor in one expression) pays the reduction and the two
// polynomials once, since the compiler merges the equal computations.  Exactly odd / even in y.
// Only IEEE single operations with explicit fused multiply-adds: the same bits on the host and on
// the device.  Against glibc's sinf / cosf over every |y| < 120 (tests/native/devmath_check.c,
// exhaustive): at most 2 ulp; sine 99.1 % equal, cosine 98.9 %, 2 ulp on fewer than 900 arguments
// each.  Larger arguments take cta_sincosf.
CTA_FN float cta_sincosf_f32(float y, int want_cos) {
    const float k = __builtin_rintf(y * 0x1.45f306p-1f);          // y * 2 / pi
    float r = CTA_FMAF(k, -0x1.921fp+0f, y);
    r = CTA_FMAF(k, -0x1.6a88p-17f, r);
    r = CTA_FMAF(k, -0x1.0b4612p-34f, r);
    const float s = r * r;
    float ps = CTA_FMAF(s, -0x1.994e02p-13f, 0x1.11075ep-7f);
    ps = CTA_FMAF(ps, s, -0x1.555546p-3f);
    const float sn = CTA_FMAF(r * s, ps, r);
    float pc = CTA_FMAF(s, 0x1.99337cp-16f, -0x1.6c087cp-10f);
    pc = CTA_FMAF(pc, s, 0x1.55553ep-5f);
    pc = CTA_FMAF(pc, s, -0.5f);
    const float cs = CTA_FMAF(pc, s, 1.0f);
    const int32_t ki = (int32_t)k;
    // quadrants 0..3: sine = sn, cs, -sn, -cs; cosine = cs, -sn, -cs, sn
    const float v = ((ki & 1) != want_cos) ? cs : sn;
    const uint32_t quadrant = (uint32_t)ki + (uint32_t)want_cos;
    const float t = cta_u2f(cta_f2u(v) ^ ((quadrant << 30) & 0x80000000u));
    return (!want_cos && y == 0.0f) ? y : t;                      // sin(-0) = -0 (the sums above turn it into +0)
}

// ---- exp for doubles: glibc's algorithm (sysdeps/ieee754/dbl-64/e_exp.c, the ARM optimized-routines
// exp with a 128-entry table of 2^(k/128) and a degree-5 polynomial), with the fused multiply-adds of
// glibc's FMA build written out.  cta_exp64_tab[2k] = the relative tail T of 2^(k/128) = H (1 + T)
// (H the nearest double), [2k+1] = bits(H) - (k << 52) / 128; computed here with 400-bit integer
// roots.  Against the installed glibc 2.35: no mismatch on 3 * 10^8 random arguments over the whole
// range, the subnormal results and both thresholds included (tests/native/exp64_check.c).
CTA_TAB_SPACE uint64_t cta_exp64_tab[256] = {
    0x0000000000000000ULL, 0x3ff0000000000000ULL, 0x3c9b3b4f1a88bf6eULL, 0x3feff63da9fb3335ULL,
    0xbc7160139cd8dc5dULL, 0x3fefec9a3e778061ULL, 0xbc905e7a108766d1ULL, 0x3fefe315e86e7f85ULL,
    0x3c8cd2523567f613ULL, 0x3fefd9b0d3158574ULL, 0xbc8bce8023f98efaULL, 0x3fefd06b29ddf6deULL,
    0x3c60f74e61e6c861ULL, 0x3fefc74518759bc8ULL, 0x3c90a3e45b33d399ULL, 0x3fefbe3ecac6f383ULL,
    0x3c979aa65d837b6dULL, 0x3fefb5586cf9890fULL, 0x3c8eb51a92fdeffcULL, 0x3fefac922b7247f7ULL,
    0x3c3ebe3d702f9cd1ULL, 0x3fefa3ec32d3d1a2ULL, 0xbc6a033489906e0bULL, 0x3fef9b66affed31bULL,
    0xbc9556522a2fbd0eULL, 0x3fef9301d0125b51ULL, 0xbc5080ef8c4eea55ULL, 0x3fef8abdc06c31ccULL,
    0xbc91c923b9d5f416ULL, 0x3fef829aaea92de0ULL, 0x3c80d3e3e95c55afULL, 0x3fef7a98c8a58e51ULL,
    0xbc801b15eaa59348ULL, 0x3fef72b83c7d517bULL, 0xbc8f1ff055de323dULL, 0x3fef6af9388c8deaULL,
    0x3c8b898c3f1353bfULL, 0x3fef635beb6fcb75ULL, 0xbc96d99c7611eb26ULL, 0x3fef5be084045cd4ULL,
    0x3c9aecf73e3a2f60ULL, 0x3fef54873168b9aaULL, 0xbc8fe782cb86389dULL, 0x3fef4d5022fcd91dULL,
    0x3c8a6f4144a6c38dULL, 0x3fef463b88628cd6ULL, 0x3c807a05b0e4047dULL, 0x3fef3f49917ddc96ULL,
    0x3c968efde3a8a894ULL, 0x3fef387a6e756238ULL, 0x3c875e18f274487dULL, 0x3fef31ce4fb2a63fULL,
    0x3c80472b981fe7f2ULL, 0x3fef2b4565e27cddULL, 0xbc96b87b3f71085eULL, 0x3fef24dfe1f56381ULL,
    0x3c82f7e16d09ab31ULL, 0x3fef1e9df51fdee1ULL, 0xbc3d219b1a6fbffaULL, 0x3fef187fd0dad990ULL,
    0x3c8b3782720c0ab4ULL, 0x3fef1285a6e4030bULL, 0x3c6e149289cecb8fULL, 0x3fef0cafa93e2f56ULL,
    0x3c834d754db0abb6ULL, 0x3fef06fe0a31b715ULL, 0x3c864201e2ac744cULL, 0x3fef0170fc4cd831ULL,
    0x3c8fdd395dd3f84aULL, 0x3feefc08b26416ffULL, 0xbc86a3803b8e5b04ULL, 0x3feef6c55f929ff1ULL,
    0xbc924aedcc4b5068ULL, 0x3feef1a7373aa9cbULL, 0xbc9907f81b512d8eULL, 0x3feeecae6d05d866ULL,
    0xbc71d1e83e9436d2ULL, 0x3feee7db34e59ff7ULL, 0xbc991919b3ce1b15ULL, 0x3feee32dc313a8e5ULL,
    0x3c859f48a72a4c6dULL, 0x3feedea64c123422ULL, 0xbc9312607a28698aULL, 0x3feeda4504ac801cULL,
    0xbc58a78f4817895bULL, 0x3feed60a21f72e2aULL, 0xbc7c2c9b67499a1bULL, 0x3feed1f5d950a897ULL,
    0x3c4363ed60c2ac11ULL, 0x3feece086061892dULL, 0x3c9666093b0664efULL, 0x3feeca41ed1d0057ULL,
    0x3c6ecce1daa10379ULL, 0x3feec6a2b5c13cd0ULL, 0x3c93ff8e3f0f1230ULL, 0x3feec32af0d7d3deULL,
    0x3c7690cebb7aafb0ULL, 0x3feebfdad5362a27ULL, 0x3c931dbdeb54e077ULL, 0x3feebcb299fddd0dULL,
    0xbc8f94340071a38eULL, 0x3feeb9b2769d2ca7ULL, 0xbc87deccdc93a349ULL, 0x3feeb6daa2cf6642ULL,
    0xbc78dec6bd0f385fULL, 0x3feeb42b569d4f82ULL, 0xbc861246ec7b5cf6ULL, 0x3feeb1a4ca5d920fULL,
    0x3c93350518fdd78eULL, 0x3feeaf4736b527daULL, 0x3c7b98b72f8a9b05ULL, 0x3feead12d497c7fdULL,
    0x3c9063e1e21c5409ULL, 0x3feeab07dd485429ULL, 0x3c34c7855019c6eaULL, 0x3feea9268a5946b7ULL,
    0x3c9432e62b64c035ULL, 0x3feea76f15ad2148ULL, 0xbc8ce44a6199769fULL, 0x3feea5e1b976dc09ULL,
    0xbc8c33c53bef4da8ULL, 0x3feea47eb03a5585ULL, 0xbc845378892be9aeULL, 0x3feea34634ccc320ULL,
    0xbc93cedd78565858ULL, 0x3feea23882552225ULL, 0x3c5710aa807e1964ULL, 0x3feea155d44ca973ULL,
    0xbc93b3efbf5e2228ULL, 0x3feea09e667f3bcdULL, 0xbc6a12ad8734b982ULL, 0x3feea012750bdabfULL,
    0xbc6367efb86da9eeULL, 0x3fee9fb23c651a2fULL, 0xbc80dc3d54e08851ULL, 0x3fee9f7df9519484ULL,
    0xbc781f647e5a3ecfULL, 0x3fee9f75e8ec5f74ULL, 0xbc86ee4ac08b7db0ULL, 0x3fee9f9a48a58174ULL,
    0xbc8619321e55e68aULL, 0x3fee9feb564267c9ULL, 0x3c909ccb5e09d4d3ULL, 0x3feea0694fde5d3fULL,
    0xbc7b32dcb94da51dULL, 0x3feea11473eb0187ULL, 0x3c94ecfd5467c06bULL, 0x3feea1ed0130c132ULL,
    0x3c65ebe1abd66c55ULL, 0x3feea2f336cf4e62ULL, 0xbc88a1c52fb3cf42ULL, 0x3feea427543e1a12ULL,
    0xbc9369b6f13b3734ULL, 0x3feea589994cce13ULL, 0xbc805e843a19ff1eULL, 0x3feea71a4623c7adULL,
    0xbc94d450d872576eULL, 0x3feea8d99b4492edULL, 0x3c90ad675b0e8a00ULL, 0x3feeaac7d98a6699ULL,
    0x3c8db72fc1f0eab4ULL, 0x3feeace5422aa0dbULL, 0xbc65b6609cc5e7ffULL, 0x3feeaf3216b5448cULL,
    0x3c7bf68359f35f44ULL, 0x3feeb1ae99157736ULL, 0xbc93091fa71e3d83ULL, 0x3feeb45b0b91ffc6ULL,
    0xbc5da9b88b6c1e29ULL, 0x3feeb737b0cdc5e5ULL, 0xbc6c23f97c90b959ULL, 0x3feeba44cbc8520fULL,
    0xbc92434322f4f9aaULL, 0x3feebd829fde4e50ULL, 0xbc85ca6cd7668e4bULL, 0x3feec0f170ca07baULL,
    0x3c71affc2b91ce27ULL, 0x3feec49182a3f090ULL, 0x3c6dd235e10a73bbULL, 0x3feec86319e32323ULL,
    0xbc87c50422622263ULL, 0x3feecc667b5de565ULL, 0x3c8b1c86e3e231d5ULL, 0x3feed09bec4a2d33ULL,
    0xbc91bbd1d3bcbb15ULL, 0x3feed503b23e255dULL, 0x3c90cc319cee31d2ULL, 0x3feed99e1330b358ULL,
    0x3c8469846e735ab3ULL, 0x3feede6b5579fdbfULL, 0xbc82dfcd978e9db4ULL, 0x3feee36bbfd3f37aULL,
    0x3c8c1a7792cb3387ULL, 0x3feee89f995ad3adULL, 0xbc907b8f4ad1d9faULL, 0x3feeee07298db666ULL,
    0xbc55c3d956dcaebaULL, 0x3feef3a2b84f15fbULL, 0xbc90a40e3da6f640ULL, 0x3feef9728de5593aULL,
    0xbc68d6f438ad9334ULL, 0x3feeff76f2fb5e47ULL, 0xbc91eee26b588a35ULL, 0x3fef05b030a1064aULL,
    0x3c74ffd70a5fddcdULL, 0x3fef0c1e904bc1d2ULL, 0xbc91bdfbfa9298acULL, 0x3fef12c25bd71e09ULL,
    0x3c736eae30af0cb3ULL, 0x3fef199bdd85529cULL, 0x3c8ee3325c9ffd94ULL, 0x3fef20ab5fffd07aULL,
    0x3c84e08fd10959acULL, 0x3fef27f12e57d14bULL, 0x3c63cdaf384e1a67ULL, 0x3fef2f6d9406e7b5ULL,
    0x3c676b2c6c921968ULL, 0x3fef3720dcef9069ULL, 0xbc808a1883ccb5d2ULL, 0x3fef3f0b555dc3faULL,
    0xbc8fad5d3ffffa6fULL, 0x3fef472d4a07897cULL, 0xbc900dae3875a949ULL, 0x3fef4f87080d89f2ULL,
    0x3c74a385a63d07a7ULL, 0x3fef5818dcfba487ULL, 0xbc82919e2040220fULL, 0x3fef60e316c98398ULL,
    0x3c8e5a50d5c192acULL, 0x3fef69e603db3285ULL, 0x3c843a59ac016b4bULL, 0x3fef7321f301b460ULL,
    0xbc82d52107b43e1fULL, 0x3fef7c97337b9b5fULL, 0xbc892ab93b470dc9ULL, 0x3fef864614f5a129ULL,
    0x3c74b604603a88d3ULL, 0x3fef902ee78b3ff6ULL, 0x3c83c5ec519d7271ULL, 0x3fef9a51fbc74c83ULL,
    0xbc8ff7128fd391f0ULL, 0x3fefa4afa2a490daULL, 0xbc8dae98e223747dULL, 0x3fefaf482d8e67f1ULL,
    0x3c8ec3bc41aa2008ULL, 0x3fefba1bee615a27ULL, 0x3c842b94c3a9eb32ULL, 0x3fefc52b376bba97ULL,
    0x3c8a64a931d185eeULL, 0x3fefd0765b6e4540ULL, 0xbc8e37bae43be3edULL, 0x3fefdbfdad9cbe14ULL,
    0x3c77893b4d91cd9dULL, 0x3fefe7c1819e90d8ULL, 0x3c5305c14160cc89ULL, 0x3feff3c22b8f71f1ULL,
};
// results near the overflow threshold or in the subnormal range (|x| >= 512)
CTA_FN double cta_exp64_special(double tmp, uint64_t sbits, uint64_t ki) {
    if ((ki & 0x80000000u) == 0) {                 // k > 0: the exponent of scale might have overflowed by <= 460
        sbits -= (uint64_t)1009 << 52;
        const double scale = cta_u2d(sbits);
        return 0x1p1009 * CTA_FMA(scale, tmp, scale);
    }
    sbits += (uint64_t)1022 << 52;                 // k < 0: care in the subnormal range
    const double scale = cta_u2d(sbits);
    const double p = scale * tmp;
    double y = scale + p;
    if (y < 1.0) {                                 // round y to the right precision before scaling it down
        double lo = scale - y + p;
        const double hi = 1.0 + y;
        lo = 1.0 - hi + y + lo;
        y = (hi + lo) - 1.0;
        if (y == 0.0) y = 0.0;                     // no -0 from a sum that rounded down
    }
    return 0x1p-1022 * y;
}
CTA_FN double cta_exp64(double x, const uint64_t* tab) {
    uint32_t abstop = (uint32_t)(cta_d2u(x) >> 52) & 0x7ffu;
    if (abstop - 0x3c9u >= 0x408u - 0x3c9u) {      // |x| < 2^-54, |x| >= 512, inf or NaN
        if (abstop - 0x3c9u >= 0x80000000u) return 1.0 + x;
        if (abstop >= 0x409u) {                    // |x| >= 1024
            if (cta_d2u(x) == 0xfff0000000000000ull) return 0.0;
            if (abstop >= 0x7ffu) return 1.0 + x;
            return (cta_d2u(x) >> 63) ? 0.0 : __builtin_huge_val();
        }
        abstop = 0;                                // large |x|: the scale needs the special case
    }
    double kd = CTA_FMA(0x1.71547652b82fep0 * 128.0, x, 0x1.8p52);
    const uint64_t ki = cta_d2u(kd);
    kd -= 0x1.8p52;
    const double r = CTA_FMA(kd, -0x1.cf79abc9e3b3ap-47, CTA_FMA(kd, -0x1.62e42fefa0000p-8, x));
    const uint64_t idx = 2 * (ki % 128);
    const uint64_t top = ki << (52 - 7);
    const double tail = cta_u2d(tab[idx]);
    const uint64_t sbits = tab[idx + 1] + top;
    const double r2 = r * r;
    const double tmp = CTA_FMA(r2 * r2, CTA_FMA(r, 0x1.1111167a4d017p-7, 0x1.55555cf172b91p-5),
                               CTA_FMA(r2, CTA_FMA(r, 0x1.555555555543cp-3, 0x1.ffffffffffdbdp-2), tail + r));
    if (abstop == 0) return cta_exp64_special(tmp, sbits, ki);
    const double scale = cta_u2d(sbits);
    return CTA_FMA(scale, tmp, scale);
}

#if defined(__HIPCC__)
// ----------------------------------------------------------------------------------------------
// Single-precision exponential for the kernels whose time the double-precision one above would set
// (row softmax, the cross-entropy gradients, fused expressions): exp(d) = 2^z * exp(d - z ln 2) with
// z = d * log2(e) rounded to float and 2^z from the hardware instruction (accurate to 1 ulp).  What
// the rounded z misses of d is recovered by two fused multiply-adds against ln 2 split in two floats
// (t = d - z ln 2, |t| < 1e-5, known to ~1e-12) and put back as the first-order factor 1 + t (the
// next term is below 1e-10).  Results stay within 2 ulp of expf (measured: 1).  NaN stays NaN,
// arguments below -150 give the hardware's 2^-216 = 0, results that would be subnormal are flushed
// to zero by the instruction.
__device__ __forceinline__ static float cta_exp_hw_nonpos(float d) {
    const float dc = (d < -150.0f) ? -150.0f : d;              // also keeps -inf out of inf - inf below
    const float z = dc * 0x1.715476p+0f;
    const float e = __builtin_amdgcn_exp2f(z);
    float t = __fmaf_rn(z, -0x1.62e4p-1f, dc);                  // ln 2 = 0x1.62e4p-1 + 0x1.7f7d1cp-20 (the first exact in 16 bits)
    t = __fmaf_rn(z, -0x1.7f7d1cp-20f, t);
    return __fmaf_rn(e, t, e);
}
// The same for any argument: overflow gives +inf (the factor must not meet an infinite e: inf * 0).
__device__ __forceinline__ static float cta_exp_hw(float d) {
    const float dc = (d < -150.0f) ? -150.0f : ((d > 90.0f) ? 90.0f : d);
    const float z = dc * 0x1.715476p+0f;
    const float e = __builtin_amdgcn_exp2f(z);
    float t = __fmaf_rn(z, -0x1.62e4p-1f, dc);
    t = __fmaf_rn(z, -0x1.7f7d1cp-20f, t);
    const float r = __fmaf_rn(e, t, e);
    return (e == __builtin_huge_valf()) ? e : r;
}
// 1 / s for finite 1 <= s <= 2^126: the hardware reciprocal (1 ulp) and two Newton steps on the exact
// residual.  Checked on the host over every significand and every starting value within 1 ulp
// (tests/native/rcpcheck.c): the correctly rounded quotient, except for a significand of all ones,
// where it is the float below (1 ulp off; 1 / s sits 2^-48 above a midpoint there).
__device__ __forceinline__ static float cta_rcp_refined(float s) {
    float r = __builtin_amdgcn_rcpf(s);
    r = __fmaf_rn(__fmaf_rn(-s, r, 1.0f), r, r);
    return __fmaf_rn(__fmaf_rn(-s, r, 1.0f), r, r);
}
// Arguments for which cta_sigmoid_f32 below is not valid, or not within its bound: NaN, x > 128 (the
// scaled argument overflows), and x < -16.625, where e^-x reaches 2^24: in [2^24, 2^25) the sum 1 + e is
// a tie for every e, two exponentials one ulp apart can round to sums TWO ulps apart, and the
// quotient moves by up to four of its ulps (seen on the device: x in [-16.93, -16.64]).  Beyond that
// binade the bound would hold again, but such sigmoids are below 6e-8; they all take the
// double-precision routine.
__device__ __forceinline__ static int cta_sigmoid_is_rare(float x) { return !(x >= -16.625f && x <= 128.0f); }
// Single-precision sigmoid by the reference's formula 1 / (1 + e^-x) for -16.625 <= x <= 128: the
// exponential above (within 1 ulp of expf), the same rounded sum, and the reciprocal above.  Against the same
// formula on expf and an exact division (what the exact mode returns): within 2 ulp.  Why: one ulp of
// the exponential moves the rounded sum s = 1 + e by at most one of its own ulps (ulp(e) <= ulp(s),
// rounding is monotonic, and for e < 2^24 at most one of two neighbouring sums is a tie).  With
// s = m 2^k, 1 <= m < 2, neighbouring sums give quotients 2^-23 / m^2
// (relative to 2^-k) apart while floats at 1 / s are 2^-24 apart: less than two ulps, so the two
// correctly rounded quotients differ by at most 2.  Where the reciprocal above is the float below
// the correct one (m all ones), the neighbours of s are 2^(k+1), whose quotient is that very float,
// and s - ulp, whose quotient rounds to the float above it: 0 and 1 ulp.
__device__ __forceinline__ static float cta_sigmoid_f32(float x) {
    const float z = x * -0x1.715476p+0f;
    const float e = __builtin_amdgcn_exp2f(z);
    float t = __fmaf_rn(z, -0x1.62e4p-1f, -x);
    t = __fmaf_rn(z, -0x1.7f7d1cp-20f, t);
    const float s = 1.0f + __fmaf_rn(e, t, e);
    return cta_rcp_refined(s);
}
#endif

#endif  // CTORCH_AMD_DEVMATH_H
