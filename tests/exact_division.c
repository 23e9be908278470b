/*
 * Exhaustive check of the division shortcut used by the HIP kernels:
 *     q = fma(f, r, f * r_lo),  r = RN(1/s),  r_lo = RN(fma(-s, r, 1) / s)
 * equals RN(f / s) for every finite e4m3 value f (all 126 positive magnitudes,
 * both signs) and every binary32 scale s = 1.m x 2^e.  All 2^23 mantissas are
 * run at e = 0; because every step scales exactly by powers of two while no
 * intermediate is subnormal, the boundary exponents e = -64 and e = +64 (the
 * ends of the range the kernels accept) are run too with the extreme codes.
 * The kernels compute r_lo without the second divide, as one Newton step on
 * e * r with e = fma(-s, r, 1):  lo = e * r,  r_lo = fma(fma(-s, lo, e), r, lo);
 * the same loops check that this is RN(e / s) bit for bit.
 * Prints the number of mismatches; exit status 0 iff there are none.
 * Build: gcc -O2 -ffp-contract=off exact_division.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

int main(void)
{
    float fv[126];
    int nf = 0;
    for (int c = 1; c < 127; c++) {
        int E = (c >> 3) & 15, M = c & 7;
        fv[nf++] = E ? ldexpf(1.0f + M / 8.0f, E - 7) : ldexpf(M / 8.0f, -6);
    }
    long bad = 0, total = 0;
    const int exps[3] = {0, -64, 64};
    for (int ei = 0; ei < 3; ei++) {
        for (uint32_t man = 0; man < (1u << 23); man++) {
            const float s = u2f(((uint32_t)(127 + exps[ei]) << 23) | man);
            const float r = 1.0f / s;
            const float e = fmaf(-s, r, 1.0f);
            const float r_lo = e / s;
            const float lo = e * r;
            if (fmaf(fmaf(-s, lo, e), r, lo) != r_lo) bad++;
            total++;
            for (int i = 0; i < nf; i++) {
                if (ei != 0 && i >= 8 && i < nf - 8) continue; /* extremes only */
                const float f = fv[i];
                if (fmaf(f, r, f * r_lo) != f / s) bad++;
                if (fmaf(-f, r, -f * r_lo) != -f / s) bad++;
                total += 2;
            }
        }
    }
    printf("checked %ld quotients, %ld mismatches\n", total, bad);
    return bad != 0;
}
