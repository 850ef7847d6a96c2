/* CPU check of the division-free quotient used by the FP8 row-encode kernel.
 *
 * The kernel computes q = x / s (s = rowmax / 448) as
 *     y = 1 / s (IEEE);  q0 = x * y;  r = fma(-s, q0, x);  q = fma(r, y, q0)
 * and relies on q being the correctly rounded fp32 quotient whenever it matters for the E4M3
 * code (|q| >= 2^-12).  x and rowmax are bf16 values.  This program compares the sequence
 * with the IEEE divide for every bf16 x <= rowmax, for every `stride`-th bf16 rowmax whose
 * biased exponent lies in [60, 190] (the window in which the kernel uses the fast path).
 * usage: markstein_check <stride>   (stride 1 = exhaustive, about a minute on 8 cores)
 * prints "checked <n> mismatches <m>".
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

int main(int argc, char** argv) {
    int stride = argc > 1 ? atoi(argv[1]) : 97;
    long long bad = 0, total = 0;
#pragma omp parallel for reduction(+ : bad, total) schedule(dynamic, 16)
    for (int ab = 0; ab < 0x7f80; ab += stride) {
        int e = (ab >> 7) & 0xff;
        if (e < 60 || e > 190) continue;
        float amax = u2f((uint32_t)ab << 16);
        float s = amax / 448.0f, y = 1.0f / s;
        for (uint32_t xb = 0; xb <= (uint32_t)ab; xb++) {
            float x = u2f(xb << 16);
            float q0 = x * y;
            float q = fmaf(fmaf(-s, q0, x), y, q0);
            float ref = x / s;
            total++;
            if (fabsf(ref) >= 0x1p-12f && f2u(q) != f2u(ref)) bad++;
        }
    }
    printf("checked %lld mismatches %lld\n", total, bad);
    return bad != 0;
}
