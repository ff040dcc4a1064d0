/* Host check of an identity the device quantizer (pocketllm_amd/csrc/pllm_device.h, quantize4) relies on:
 * for EVERY finite positive float32 a, with c = fl(1 / 127),
 *     q0 = fl(a * c);  r = fma(-q0, 127, a);  fma(r, c, q0)  ==  the correctly rounded quotient a / 127.
 * Exhaustive over all 2^31 - 2^23 bit patterns; prints the number of mismatches (0 expected) and returns it as exit status.
 * Build: gcc -O2 -mfma -ffp-contract=off -fopenmp quantizer_div127.c -lm */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

int main(void) {
    const float c = 1.0f / 127.0f;
    long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (int64_t u = 1; u < 0x7f800000ll; ++u) {
        const uint32_t bits = (uint32_t)u;
        float a;
        memcpy(&a, &bits, 4);
        const float want = a / 127.0f;
        const float q0 = a * c;
        const float r = fmaf(-q0, 127.0f, a);
        const float q1 = fmaf(r, c, q0);
        if (q1 != want) ++bad;
    }
    printf("%ld\n", bad);
    return bad != 0;
}
