/*
 * wr_math.c — scalar math for the CPU ops of the host engine.
 *
 * These follow the reference's polynomial forms operation for operation
 * (reference: src/core/mathx.c:37-57 exp, :72-86 log, :98-110 sqrt,
 * :124-147 sin/cos) because RMSNorm, SiLU and RoPE feed the attention path:
 * using libm here would shift the K/V rows that reach the cache by a few ulp
 * and with them the greedy token stream that is compared step for step.
 * Build without FMA contraction (-ffp-contract=off) for the same reason.
 */
#include "wr_host.h"

#include <string.h>

static inline uint32_t as_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float as_float(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Split x = k ln2 + r (k nearest integer), fifth-order series in r, then add k
 * to the exponent field.  Clamped to [-88, 88]. */
float wrh_exp(float x)
{
    if (x < -88.0f) return 0.0f;
    if (x > 88.0f) return 1e38f;
    const float ln2 = 0.6931471805599453f;
    const int k = (int)(x / ln2 + (x >= 0 ? 0.5f : -0.5f));
    const float r = x - (float)k * ln2;
    const float r2 = r * r;
    float e = 1.0f + r + r2 * 0.5f + r2 * r * (1.0f / 6.0f) + r2 * r2 * (1.0f / 24.0f) +
              r2 * r2 * r * (1.0f / 120.0f);
    if (k >= -126 && k <= 127) e = as_float(as_bits(e) + ((uint32_t)k << 23));
    return e;
}

/* ln(m 2^e) = ln m + e ln2, ln m from four terms of the atanh series. */
float wrh_log(float x)
{
    if (x <= 0.0f) return -1e38f;
    const uint32_t u = as_bits(x);
    const int e = (int)((u >> 23) & 0xFF) - 127;
    const float m = as_float((u & 0x007FFFFFu) | 0x3F800000u);
    const float t = (m - 1.0f) / (m + 1.0f);
    const float t2 = t * t;
    const float lnm =
        2.0f * t * (1.0f + t2 * (1.0f / 3.0f + t2 * (1.0f / 5.0f + t2 * (1.0f / 7.0f))));
    return lnm + (float)e * 0.6931471805599453f;
}

/* Exponent-halving seed and four Newton steps. */
float wrh_sqrt(float x)
{
    if (x <= 0) return 0;
    float g = as_float((as_bits(x) + 0x3f800000u) >> 1);
    g = 0.5f * (g + x / g);
    g = 0.5f * (g + x / g);
    g = 0.5f * (g + x / g);
    g = 0.5f * (g + x / g);
    return g;
}

static float wrap_pi(float x)
{
    const float pi = 3.14159265358979f, two_pi = 6.28318530717958f;
    while (x > pi) x -= two_pi;
    while (x < -pi) x += two_pi;
    return x;
}

float wrh_sin(float x)
{
    x = wrap_pi(x);
    const float x2 = x * x, x3 = x2 * x, x5 = x3 * x2, x7 = x5 * x2;
    return x - x3 * (1.0f / 6.0f) + x5 * (1.0f / 120.0f) - x7 * (1.0f / 5040.0f);
}

float wrh_cos(float x)
{
    x = wrap_pi(x);
    const float x2 = x * x, x4 = x2 * x2, x6 = x4 * x2;
    return 1.0f - x2 * 0.5f + x4 * (1.0f / 24.0f) - x6 * (1.0f / 720.0f);
}

/* reference: src/core/mathx.c:158-161 (2/(1+e^-2x) rounds once) */
float wrh_tanh(float x)
{
    return 2.0f / (1.0f + wrh_exp(-2.0f * x)) - 1.0f;
}
