/* Host check of ctorch_amd/csrc/devmath.h against the installed glibc: counts the floats for
 * which the device algorithms (compiled here for the CPU, unchanged) return different bits from
 * expf / sinf / cosf / logf, and the worst distance of the tangent from glibc's tanf (not the same
 * algorithm: at most 1 ulp) and of the single-precision sine / cosine pair from sinf / cosf (at most 2
 * ulp, |x| < 120; also that the pair is exactly odd / even).  Usage: devmath_check STRIDE  (1 = every one of the 2^32 bit patterns).
 * Prints one line per function: name, inputs tested, mismatches, worst ulp distance
 * (expf_pair: exp(x) and exp(-x) from the shared reduction, against expf(x) and expf(-x)). */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "../../ctorch_amd/csrc/devmath.h"

static int64_t ulpkey(float f) {
    int32_t i = (int32_t)cta_f2u(f);
    return i < 0 ? -(int64_t)(i & 0x7fffffff) : i;
}
static int differs(float a, float b, int64_t* ulp) {
    if (a != a && b != b) return 0;
    if (cta_f2u(a) == cta_f2u(b)) return 0;
    int64_t d = ulpkey(a) - ulpkey(b);
    *ulp = d < 0 ? -d : d;
    return 1;
}

int main(int argc, char** argv) {
    uint64_t stride = argc > 1 ? strtoull(argv[1], 0, 10) : 1;
    if (stride == 0) stride = 1;
    uint64_t n = 0, bad[8] = {0, 0, 0, 0, 0, 0, 0, 0}, covered[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t worst[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma omp parallel for reduction(+ : n, bad[:8], covered[:8]) reduction(max : worst[:8]) schedule(static)
    for (uint64_t u = 0; u < (1ULL << 32); u += stride) {
        float x = cta_u2f((uint32_t)u);
        int64_t d = 0;
        ++n;
        ++covered[0];
        if (differs(cta_expf_tab(x, cta_exp2_tab), expf(x), &d)) {
            ++bad[0];
            if (d > worst[0]) worst[0] = d;
        }
        if (!(x > 0.0f) && differs(cta_expf_nonpos(x, cta_exp2_tab), expf(x), &d)) {   /* x <= 0 or NaN */
            ++bad[0];
            if (d > worst[0]) worst[0] = d;
        }
        float ep, en;
        cta_expf_pair(x, cta_exp2_tab, &ep, &en);
        ++covered[3];
        if (differs(ep, expf(x), &d) || differs(en, expf(-x), &d)) {
            ++bad[3];
            if (d > worst[3]) worst[3] = d;
        }
        ++covered[1];
        if (differs(cta_sincosf(x, 0, cta_inv_pio4), sinf(x), &d)) {
            ++bad[1];
            if (d > worst[1]) worst[1] = d;
        }
        ++covered[2];
        if (differs(cta_sincosf(x, 1, cta_inv_pio4), cosf(x), &d)) {
            ++bad[2];
            if (d > worst[2]) worst[2] = d;
        }
        ++covered[4];
        if (differs(cta_logf(x, cta_log_tab), logf(x), &d)) {
            ++bad[4];
            if (d > worst[4]) worst[4] = d;
        }
        ++covered[5];
        if (differs(cta_tanf(x, cta_inv_pio4), tanf(x), &d)) {
            if (d > 1) ++bad[5];                   /* a different algorithm: 1 ulp apart is expected */
            if (d > worst[5]) worst[5] = d;
        }
        if (!cta_sincos_is_rare(x)) {               /* the single-precision pair: |x| < 120, at most 2 ulp */
            ++covered[6];
            if (differs(cta_sincosf_f32(x, 0), sinf(x), &d)) {
                if (d > 2 || d == 0) ++bad[6];     /* d == 0: zeros of opposite sign */
                if (d > worst[6]) worst[6] = d;
            }
            ++covered[7];
            if (differs(cta_sincosf_f32(x, 1), cosf(x), &d)) {
                if (d > 2 || d == 0) ++bad[7];
                if (d > worst[7]) worst[7] = d;
            }
            /* exactly odd / even: the fused-expression compiler forms sin(-x), cos(-x) from sin(x), cos(x) */
            if (cta_f2u(cta_sincosf_f32(-x, 0)) != (cta_f2u(cta_sincosf_f32(x, 0)) ^ 0x80000000u)) ++bad[6];
            if (cta_f2u(cta_sincosf_f32(-x, 1)) != cta_f2u(cta_sincosf_f32(x, 1))) ++bad[7];
        }
    }
    const char* names[8] = {"expf", "sinf", "cosf", "expf_pair", "logf", "tanf(>1ulp)", "sinf_f32(>2ulp)", "cosf_f32(>2ulp)"};
    for (int k = 0; k < 8; ++k)
        printf("%s tested %llu mismatches %llu worst_ulp %lld\n", names[k], (unsigned long long)covered[k],
               (unsigned long long)bad[k], (long long)worst[k]);
    return 0;
}
