// Compares the restated float routines (glades-ml_amd/csrc/libm_exact.h) with this machine's C
// library: libm_check <stride> [first] visits the floats whose bit patterns are first, first+stride, ...
// and prints the number of inputs on which each routine differs (NaN results count as equal).
// With stride 1 it is the exhaustive comparison (about half a minute on 8 cores).
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "../glades-ml_amd/csrc/libm_exact.h"

static bool same(float a, float b) { return glm_f2u(a) == glm_f2u(b) || (a != a && b != b); }

int main(int argc, char** argv)
{
    const long long stride = argc > 1 ? atoll(argv[1]) : 61;
    const long long first = argc > 2 ? atoll(argv[2]) : 0;
    if (stride < 1) return 2;
    long long bad_tanh = 0, bad_exp = 0, bad_log = 0, bad_expm1 = 0, n = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad_tanh, bad_exp, bad_log, bad_expm1, n)
    for (long long i = first; i < (1LL << 32); i += stride) {
        const float x = glm_u2f((uint32_t)i);
        if (!same(glm_tanhf(x), tanhf(x))) ++bad_tanh;
        if (!same(glm_expf(x), expf(x))) ++bad_exp;
        if (!same(glm_logf(x), logf(x))) ++bad_log;
        if (!same(glm_expm1f(x), expm1f(x))) ++bad_expm1;
        ++n;
    }
    printf("inputs %lld tanhf %lld expf %lld logf %lld expm1f %lld\n", n, bad_tanh, bad_exp, bad_log, bad_expm1);
    return 0;
}
