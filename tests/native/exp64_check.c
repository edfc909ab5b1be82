/* Host check of cta_exp64 (ctorch_amd/csrc/devmath.h, the exponential of the double softmax) against
 * the installed glibc's exp: random arguments over the whole range, around zero, at the overflow
 * threshold and through the subnormal results, plus special values.
 * Usage: exp64_check N   (arguments per region; four regions and their mirror set).
 * Prints: tested N mismatches M */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "../../ctorch_amd/csrc/devmath.h"

int main(int argc, char** argv) {
    long n = argc > 1 ? atol(argv[1]) : 10000000;
    long bad = 0, tested = 0;
#pragma omp parallel for reduction(+ : bad, tested) schedule(static)
    for (long i = 0; i < n; ++i) {
        uint64_t s = 88172645463325252ull + 0x9E3779B97F4A7C15ull * (uint64_t)i;
        s ^= s >> 30; s *= 0xBF58476D1CE4E5B9ull; s ^= s >> 27; s *= 0x94D049BB133111EBull; s ^= s >> 31;
        const double u = (double)(s >> 11) * (1.0 / 9007199254740992.0);
        const double xs[8] = {-745.2 + u * (709.8 + 745.2), -40.0 + 80.0 * u, -1.0 + 2.0 * u, -20.0 * u,
                              -745.2 + u * 37.5, (u - 0.5) * 0x1p-50, 709.0 + u * 0.8, -708.5 + u};
        for (int k = 0; k < 8; ++k) {
            ++tested;
            if (cta_d2u(cta_exp64(xs[k], cta_exp64_tab)) != cta_d2u(exp(xs[k]))) ++bad;
        }
    }
    const double sp[] = {0.0, -0.0, 1.0, -1.0, 709.78, 709.79, -745.1, -745.2, -708.4, -708.3, 1e-300, -1e-300,
                         INFINITY, -INFINITY, 0x1p-60, 512.0, -512.0, 1024.0, -1024.0, 0x1.62e42fefa39efp+9};
    for (unsigned k = 0; k < sizeof(sp) / sizeof(sp[0]); ++k) {
        ++tested;
        if (cta_d2u(cta_exp64(sp[k], cta_exp64_tab)) != cta_d2u(exp(sp[k]))) ++bad;
    }
    ++tested;
    if (!(cta_exp64(NAN, cta_exp64_tab) != cta_exp64(NAN, cta_exp64_tab))) ++bad;
    printf("tested %ld mismatches %ld\n", tested, bad);
    return 0;
}
