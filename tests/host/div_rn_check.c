/* CPU check of the identity behind div_rn (torsh_amd/csrc/hipq_math.h): with y = RN(1/b),
 * q0 = RN(a*y), r = fma(-q0, b, a), the value fma(r, y, q0) equals the correctly rounded a/b.
 * Every numerator significand is tried for a set of denominators (per-row scales absmax/127,
 * random significands, all-ones and near-one significands) and several exponent offsets.
 * Usage: div_rn_check [denominators] ; prints a summary, exit status 1 on any mismatch.
 * The full sweep behind the claim in the header comment is `div_rn_check 3000` (minutes). */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static float asf(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

int main(int argc, char **argv) {
    const int want = argc > 1 ? atoi(argv[1]) : 24;
    uint32_t *bs = malloc(sizeof(uint32_t) * (size_t)(want + 8));
    int nb = 0;
    uint64_t s = 88172645463325252ull;
    const uint32_t fixed[] = {0x3fffffffu, 0x3f800001u, 0x3f7fffffu, 0x3fc00000u, 0x3fb504f3u, 0x00800000u, 0x7e7fffffu};
    for (unsigned i = 0; i < sizeof(fixed) / sizeof(fixed[0]); ++i) bs[nb++] = fixed[i];
    while (nb < want + 7) {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        if (nb & 1) {
            float am = (float)((s >> 11) * (1.0 / 9007199254740992.0)) * 8.0f + 1e-3f, b = am / 127.0f;
            memcpy(&bs[nb++], &b, 4);
        } else {
            bs[nb++] = 0x3f800000u | (uint32_t)(s & 0x7fffff);
        }
    }
    unsigned long long bad = 0, total = 0;
#pragma omp parallel for reduction(+ : bad, total) schedule(dynamic)
    for (int bi = 0; bi < nb; ++bi) {
        const float b = asf(bs[bi]), y = 1.0f / b;
        const int exps[3] = {-3, 0, 6};
        for (int k = 0; k < 3; ++k) {
            float base = ldexpf(b, exps[k]);
            uint32_t ub; memcpy(&ub, &base, 4);
            const uint32_t expbits = ub & 0x7f800000u;
            if (expbits == 0 || expbits == 0x7f800000u) continue;
            for (uint32_t m = 0; m < (1u << 23); ++m) {
                const float a = asf(expbits | m), q0 = a * y, r = fmaf(-q0, b, a), q1 = fmaf(r, y, q0);
                if (q1 != a / b) ++bad;
                ++total;
            }
        }
    }
    printf("checked %llu quotients over %d denominators: %llu mismatches\n", total, nb, bad);
    free(bs);
    return bad != 0;
}
