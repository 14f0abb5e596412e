/* Scalar C restatement of the reference's quantise/pack and unpack/dequantise kernels.
 * TEST INFRASTRUCTURE ONLY: built by oracle/build.py into oracle/_build/ and loaded by
 * the tests through ctypes to pin the vectorised torch oracle (oracle/hyc_oracle.py)
 * with an independently written loop-level implementation.  Nothing shipped links it.
 *
 * The loops mirror the tile structure of the Triton kernels: a program handles one
 * 32-column block `pid_n` of one row; output byte j of the block collects, for
 * i = 0..epp-1, the element at column 32*pid_n + j + i*(32/epp), shifted by q*i
 * (operators/compress_function_kernel.py:77-112 and :166-206; zero-point forms
 * :262-301 and :345-388).
 *
 * bf16 values travel as uint16_t bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf2f(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f2bf(float f) { /* round to nearest even, as a bf16 store does */
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* x: [B,M,N] bf16, s: [N] bf16, z: [N] bf16 or NULL, q: [B,M,N*q_bit/8] bytes */
void ref_quant_pack(const uint16_t *x, const uint16_t *s, const uint16_t *z, uint8_t *q,
                    long B, long M, long N, int q_bit) {
    const int epp = 8 / q_bit;
    const int w = 32 / epp;
    const float max_val = (float)((1 << (q_bit - 1)) - 1);
    const float min_val = -(float)(1 << (q_bit - 1));
    const float total_range = (float)(1 << (q_bit - 1));
    for (long b = 0; b < B; ++b)
        for (long m = 0; m < M; ++m)
            for (long pid_n = 0; pid_n < N / 32; ++pid_n)
                for (int j = 0; j < w; ++j) {
                    unsigned byte = 0;
                    for (int i = 0; i < epp; ++i) {
                        long col = pid_n * 32 + j + (long)i * w;
                        float xv = bf2f(x[(b * M + m) * N + col]);
                        float sv = bf2f(s[col]);
                        float t = xv / sv;                 /* :103  x / s in fp32 */
                        if (z) t = t + bf2f(z[col]);       /* :292  + z */
                        t = roundf(t);                     /* libdevice round */
                        if (t < min_val) t = min_val;      /* :104-105 */
                        if (t > max_val) t = max_val;
                        t = t + total_range;               /* :106 */
                        unsigned e = isnan(t) ? 0u : (unsigned)lrintf(t); /* float2uint_rn */
                        byte |= (e << (q_bit * i)) & 0xffu;                /* :110 */
                    }
                    q[(b * M + m) * (N / epp) + pid_n * w + j] = (uint8_t)byte;
                }
}

/* inverse; xo: [B,M,N] bf16 */
void ref_unpack_dequant(const uint8_t *q, const uint16_t *s, const uint16_t *z, uint16_t *xo,
                        long B, long M, long N, int q_bit) {
    const int epp = 8 / q_bit;
    const int w = 32 / epp;
    const unsigned mask = (1u << q_bit) - 1u;
    for (long b = 0; b < B; ++b)
        for (long m = 0; m < M; ++m)
            for (long pid_n = 0; pid_n < N / 32; ++pid_n)
                for (int j = 0; j < w; ++j) {
                    unsigned byte = q[(b * M + m) * (N / epp) + pid_n * w + j];
                    for (int i = 0; i < epp; ++i) {
                        long col = pid_n * 32 + j + (long)i * w;
                        /* uint -> float -> bf16, minus 2^(q-1) in bf16 (:199-201) */
                        float v = bf2f(f2bf((float)(byte & mask)));
                        v = bf2f(f2bf(v - (float)(1 << (q_bit - 1))));
                        if (z) v = bf2f(f2bf(v - bf2f(z[col])));       /* :386 */
                        v = v * bf2f(s[col]);                            /* :202 */
                        xo[(b * M + m) * N + col] = f2bf(v);
                        byte >>= q_bit;                                  /* :205 */
                    }
                }
}
