/*
 * Exhaustive check of the division by the group size used by the reduce kernel
 * when the group size is not a power of two:
 *     r = RN(1 / d),  q0 = RN(y * r),  rem = fma(-q0, d, y),  q = fma(rem, r, q0)
 * equals RN(y / d) for every binary32 y = 1.m (all 2^23 mantissas) and every odd
 * integer d from 3 to 1023.  Every step scales exactly by powers of two while no
 * intermediate is subnormal, so the exponents of y and of d (d = odd x 2^k)
 * do not matter in that range.
 * Prints the number of mismatches; exit status 0 iff there are none.
 * Build: gcc -O2 -fopenmp -ffp-contract=off exact_quotient.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

int main(void)
{
    long bad = 0, total = 0;
#pragma omp parallel for reduction(+ : bad, total) schedule(dynamic)
    for (int d = 3; d < 1024; d += 2) {
        const float fd = (float)d;
        const float r = 1.0f / fd;
        for (uint32_t man = 0; man < (1u << 23); man++) {
            const float y = u2f((127u << 23) | man);
            const float q0 = y * r;
            const float rem = fmaf(-q0, fd, y);
            if (fmaf(rem, r, q0) != y / fd) bad++;
            total++;
        }
    }
    printf("checked %ld quotients, %ld mismatches\n", total, bad);
    return bad != 0;
}
