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
// time the double-precision routines above would set (fused expressions): the quadrant by one
// multiplication, the argument reduced against pi/2 split in three floats whose first two have 16
// significant bits (so their products with the quadrant number, below 2^8, are exact and the first
// two steps lose nothing), then the classic degree-7 / degree-8 polynomials on [-pi/4, pi/4].  Only
// IEEE single operations with explicit fused multiply-adds: the same bits on the host and on the
// device.  Within 2 ulp of glibc's sinf / cosf for every |y| < 120
// (tests/native/devmath_check.c, exhaustive); larger arguments take cta_sincosf.
CTA_FN float cta_sincosf_f32(float y, int want_cos) {
    const float nf = __builtin_rintf(y * 0x1.45f306p-1f);                  // 2 / pi
    int n = (int)nf;
    float r = CTA_FMAF(nf, -0x1.922p+0f, y);
    r = CTA_FMAF(nf, 0x1.2aeep-18f, r);
    r = CTA_FMAF(nf, 0x1.e974p-35f, r);
    const float z = r * r;
    float sp = CTA_FMAF(z, -1.9515295891e-4f, 8.3321608736e-3f);
    sp = CTA_FMAF(sp, z, -1.6666654611e-1f);
    const float sn = CTA_FMAF(r * z, sp, r);
    float cp = CTA_FMAF(z, 2.443315711809948e-5f, -1.388731625493765e-3f);
    cp = CTA_FMAF(cp, z, 4.166664568298827e-2f);
    const float c = CTA_FMAF(z * z, cp, CTA_FMAF(z, -0.5f, 1.0f));
    if (want_cos) n += 1;
    const float res = (n & 1) ? c : sn;
    return cta_u2f(cta_f2u(res) ^ ((uint32_t)(n & 2) << 30));
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
// The same with the argument held to [-150, 88], so that the result is always finite (at most e^88 =
// 1.65e38).  A NaN argument gives e^-150 = 0: callers that must return NaN for NaN select it themselves.
__device__ __forceinline__ static float cta_exp_hw_bounded(float d) {
    const float dc = __builtin_amdgcn_fmed3f(d, -150.0f, 88.0f);
    const float z = dc * 0x1.715476p+0f;
    const float e = __builtin_amdgcn_exp2f(z);
    float t = __fmaf_rn(z, -0x1.62e4p-1f, dc);
    t = __fmaf_rn(z, -0x1.7f7d1cp-20f, t);
    return __fmaf_rn(e, t, e);
}
// 1 / s for finite s >= 1: the hardware reciprocal (1 ulp) and one Newton step, within 1 ulp of
// the exactly rounded quotient.  Where 1 / s would be subnormal (s > 2^126) the result may be 0.
__device__ __forceinline__ static float cta_rcp_refined(float s) {
    const float r = __builtin_amdgcn_rcpf(s);
    const float err = __fmaf_rn(-s, r, 1.0f);
    return __fmaf_rn(err, r, r);
}
// Single-precision sigmoid by the reference's formula 1 / (1 + e^-x) on the exponential and the
// reciprocal above.  Against the same formula on expf and an exact division (what the exact mode
// returns): within 4 ulp - the sum 1 + e is rounded where its spacing is up to four times the
// spacing of the quotient, so one ulp of the exponential is worth up to four of the result - and
// below the smallest normal number (x < -87.3) possibly 0 where the exact mode has a subnormal.
__device__ __forceinline__ static float cta_sigmoid_f32(float x) {
    const float s = 1.0f + cta_exp_hw_bounded(-x);
    const float r = cta_rcp_refined(s);
    return (x != x) ? x : r;
}
// Single-precision tanh.  The reference computes (e^x - e^-x) / (e^x + e^-x); this computes the same
// function as 1 - 2 / (e^2|x| + 1) with the sign of x (one exponential, one reciprocal): within 2 ulp
// of tanh for |x| >= 1, within 1.2e-7 absolute below, where the reference's form loses its digits to
// the same cancellation.  The reference's form is inf / inf = NaN once expf(|x|) overflows, that is
// for |x| > 0x1.62e42ep+6: so is this, and NaN stays NaN.
__device__ __forceinline__ static float cta_tanh_f32(float x) {
    const float ax = __builtin_fabsf(x);
    const float s = cta_exp_hw_bounded(ax + ax) + 1.0f;
    const float v = __fmaf_rn(-2.0f, cta_rcp_refined(s), 1.0f);
    return (ax <= 0x1.62e42ep+6f) ? __builtin_copysignf(v, x) : __builtin_nanf("");
}
#endif

#endif  // CTORCH_AMD_DEVMATH_H
