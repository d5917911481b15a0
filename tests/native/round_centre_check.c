/* Host check of the short rounding sequence of the fused quantize pass (round_centre in
 * prime_amd/csrc/device_common.h): for every float q with |q| <= 628,
 *     trunc(c + copysign(0.49999997f, c)) + 128,  c = min(max(q, -128), 127)
 * equals the reference's clamp(int(roundf(q)) + 128, 0, 255)
 * (src/zeroband/C/csrc/compression.cpp:23-24).  Prints the number of values checked and of
 * mismatches; exit status 1 on a mismatch. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static inline float round_centre(float q) {
    const float c = fminf(fmaxf(q, -128.0f), 127.0f);
    return truncf(c + copysignf(0.49999997f, c));
}

static inline int reference_code(float q) {
    const float r = roundf(q);
    const int ri = (r >= -2147483648.0f && r < 2147483648.0f) ? (int)r : INT32_MIN;
    const int c = (int)((unsigned)ri + 128u);
    return c < 0 ? 0 : c > 255 ? 255 : c;
}

int main(void) {
    uint32_t lim;
    const float far = 628.0f;
    memcpy(&lim, &far, 4);
    long bad = 0, n = 0;
    for (int sign = 0; sign < 2; ++sign)
        for (uint32_t b = 0; b <= lim; ++b) {
            const uint32_t bits = b | ((uint32_t)sign << 31);
            float q;
            memcpy(&q, &bits, 4);
            if ((int)round_centre(q) + 128 != reference_code(q)) {
                if (bad < 5) printf("mismatch at %a\n", q);
                ++bad;
            }
            ++n;
        }
    printf("checked %ld mismatches %ld\n", n, bad);
    return bad != 0;
}
