/* Exhaustive check of the identity the kernels use for f32::round (half away from zero):
 *   roundf(t) == truncf(t + copysignf(h, t)),  h = largest float below 0.5,
 * over every finite float, bit for bit (signed zeros included).  Exit status 1 on any mismatch. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
int main(void) {
    unsigned long long bad = 0;
    const float h = 0x1.fffffep-2f;  /* largest float below 0.5 */
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long long i = 0; i < (1LL << 32); ++i) {
        uint32_t u = (uint32_t)i;
        float t;
        memcpy(&t, &u, 4);
        if (!(t == t) || isinf(t)) continue;
        float a = roundf(t);
        float b = truncf(t + copysignf(h, t));
        uint32_t ua, ub;
        memcpy(&ua, &a, 4);
        memcpy(&ub, &b, 4);
        if (ua != ub) {
            if (bad < 5) printf("mismatch t=%a roundf=%a trick=%a\n", t, a, b);
            ++bad;
        }
    }
    printf("%llu mismatches over all finite floats\n", bad);
    return bad != 0;
}
