/* Exhaustive host-side check of the reciprocal-based code rule used by the HIP quantiser.
 *
 * For every bf16 step s accepted by hyc_scale_is_fast and every one of the 65536 bf16
 * inputs x (NaNs and infinities included), the integer code computed by hyc_code_fast
 * (one fused multiply-add with the enlarged reciprocal, clamp, low byte), and the codes the
 * division paths compute (hyc_code_from_t, hyc_code_from_t_exact), must equal the code
 * computed from the IEEE quotient x / s with libm's roundf, for code widths 2, 4 and 8.
 * hyc_code_fast is also evaluated with the reciprocal moved to either end of the band
 * +-HYC_RECIP_SLACK (relative), which bounds what an approximate reciprocal can return.
 * Also reports how close an enlarged quotient inside the code range ever comes to a
 * half-integer (it must stay clear of one, or the rounding mode of the addition would matter).
 * Prints the number of pairs examined and the number of mismatches; exit status 0 iff none.
 *
 * Build (done by the test that runs it):
 *   gcc -O2 -fopenmp -ffp-contract=off -I<package>/csrc check_fastdiv.c -lm
 */
#include <stdio.h>
#include <stdlib.h>
#include "hyc_quant_math.h"

static int code_ieee(float x, float s, int q_bit) {
    float t = x / s;
    float half = (float)(1 << (q_bit - 1));
    t = roundf(t);
    if (t < -half) t = -half;
    if (t > half - 1.0f) t = half - 1.0f;
    t += half;
    return isnan(t) ? 0 : (int)lrintf(t);
}

int main(int argc, char **argv) {
    /* optional stride over s patterns for a quicker partial run */
    int stride = argc > 1 ? atoi(argv[1]) : 1;
    if (stride < 1) stride = 1;
    unsigned long long pairs = 0, bad = 0;
    unsigned first_bad_x = 0, first_bad_s = 0;
    double tie_gap = 1.0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : pairs, bad) reduction(min : tie_gap)
    for (int sb = 1; sb < 0x7f80; sb += stride) {
        float s = hyc_bf16_to_f32((uint16_t)sb);
        if (!hyc_scale_is_fast(s)) continue;
        float rn = hyc_recip_nudged(s);
        for (unsigned xb = 0; xb < 65536u; ++xb) {
            float x = hyc_bf16_to_f32((uint16_t)xb);
            float ti = x / s;
            ++pairs;
            int ok = 1;
            for (int q = 2; q <= 8; q *= 2) {
                const int want = code_ieee(x, s, q);
                if (hyc_code_from_t(ti, q) != want || hyc_code_from_t_exact(ti, q) != want) ok = 0;
                if (hyc_code_fast(x, rn, q) != want) ok = 0;
                /* both ends of the band that covers an approximate hardware reciprocal */
                if (hyc_code_fast(x, rn * (1.0f - HYC_RECIP_SLACK), q) != want) ok = 0;
                if (hyc_code_fast(x, rn * (1.0f + HYC_RECIP_SLACK), q) != want) ok = 0;
            }
            const double tn = (double)x * (double)rn;
            if (fabs(tn) <= 129.0) {
                const double gap = fabs(tn - floor(tn) - 0.5);
                if (gap < tie_gap) tie_gap = gap;
            }
            if (!ok) {
                ++bad;
#pragma omp critical
                if (!first_bad_s) { first_bad_s = (unsigned)sb; first_bad_x = xb; }
            }
        }
    }
    printf("pairs=%llu mismatches=%llu min_distance_to_a_tie=%.3g\n", pairs, bad, tie_gap);
    if (bad) printf("first mismatch: x=0x%04x s=0x%04x\n", first_bad_x, first_bad_s);
    return (bad || tie_gap < 1e-6) ? 1 : 0;
}
