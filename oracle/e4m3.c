/* Oracle (test infrastructure only): bit-level restatement of the reference's
 * tensorwise e4m3 quantizer, nanochat/fp8.py:81-107, in plain C with no torch.
 *
 *   amax  = max |x|                              (fp32)          fp8.py:93
 *   scale = (float)(448.0 / max((double)amax, 1e-12))            fp8.py:97-98
 *   y     = clamp((float)x * scale, -448, 448)                   fp8.py:101-102
 *   byte  = e4m3fn(y), round-to-nearest-even, subnormals to 2^-9 fp8.py:103
 *   inv   = 1.0f / scale                                         fp8.py:106
 *
 * The OCP e4m3fn format: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no
 * infinities; 0x7f/0xff are NaN; largest finite 0x7e = 448; smallest
 * subnormal 0x01 = 2^-9.
 *
 * Build: gcc -O2 -shared -fPIC -ffp-contract=off -o _build/libe4m3_oracle.so e4m3.c
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

static float bf16_bits_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Round a finite fp32 in [-448, 448] to e4m3fn, ties to even. */
uint8_t oracle_e4m3_encode(float y) {
    uint32_t u;
    memcpy(&u, &y, 4);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    float a = fabsf(y);
    if (a != a) return (uint8_t)(sign | 0x7f);
    if (a > 448.0f) a = 448.0f;            /* callers clamp first; be safe */
    if (a == 0.0f) return sign;
    int e;
    (void)frexpf(a, &e);                   /* a = m * 2^e, m in [0.5, 1) */
    int exp = e - 1;                       /* a = 1.xxx * 2^exp */
    if (exp < -6) exp = -6;                /* subnormal range shares 2^-6 */
    /* quantum = 2^(exp-3): three mantissa bits */
    float q = ldexpf(1.0f, exp - 3);
    float n = a / q;                       /* exact: power-of-two divide */
    float r = nearbyintf(n);               /* default mode = ties-to-even */
    float v = r * q;                       /* rounded magnitude (exact) */
    if (v == 0.0f) return sign;
    int e2;
    (void)frexpf(v, &e2);
    int vexp = e2 - 1;
    if (vexp < -6) {
        /* subnormal: value = mant * 2^-9, mant in 1..7 */
        int mant = (int)(v * 512.0f);
        return (uint8_t)(sign | mant);
    }
    int mant = (int)(ldexpf(v, 3 - vexp)) - 8;   /* 0..7 */
    int biased = vexp + 7;                        /* 1..15 */
    return (uint8_t)(sign | (biased << 3) | mant);
}

float oracle_e4m3_decode(uint8_t b) {
    int sign = b & 0x80;
    int e = (b >> 3) & 0xf;
    int m = b & 7;
    float v;
    if (e == 0xf && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf((float)(8 + m), e - 7 - 3);
    return sign ? -v : v;
}

static float scale_from_amax(float amax) {
    double d = (double)amax;
    if (d < 1e-12) d = 1e-12;
    return (float)(448.0 / d);
}

static void quantize_core(const float *xs, size_t n, float scale, uint8_t *out) {
    for (size_t i = 0; i < n; i++) {
        float y = xs[i] * scale;
        if (y > 448.0f) y = 448.0f;
        if (y < -448.0f) y = -448.0f;
        out[i] = oracle_e4m3_encode(y);
    }
}

/* x: n fp32 values. Writes n bytes, scale and inv_scale. */
void oracle_quantize_f32(const float *x, size_t n, uint8_t *out, float *scale_out, float *inv_out) {
    float amax = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float a = fabsf(x[i]);
        if (a > amax) amax = a;
    }
    float scale = scale_from_amax(amax);
    quantize_core(x, n, scale, out);
    *scale_out = scale;
    *inv_out = 1.0f / scale;
}

/* x: n bf16 bit patterns. */
void oracle_quantize_bf16(const uint16_t *x, size_t n, uint8_t *out, float *scale_out, float *inv_out) {
    float amax = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float a = fabsf(bf16_bits_to_f32(x[i]));
        if (a > amax) amax = a;
    }
    float scale = scale_from_amax(amax);
    for (size_t i = 0; i < n; i++) {
        float v = bf16_bits_to_f32(x[i]);
        quantize_core(&v, 1, scale, out + i);
    }
    *scale_out = scale;
    *inv_out = 1.0f / scale;
}

/* Encode with a caller-given scale (exhaustive table tests). */
void oracle_encode_bf16_with_scale(const uint16_t *x, size_t n, float scale, uint8_t *out) {
    for (size_t i = 0; i < n; i++) {
        float v = bf16_bits_to_f32(x[i]);
        quantize_core(&v, 1, scale, out + i);
    }
}
