/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Storage formats and rounding helpers shared by the C files of the CPU oracle:
 * fp16 / bf16 as raw uint16_t bit patterns, fp32 as float; conversions round to
 * nearest even. Everything is `static`: each translation unit gets its own copy.
 */
#ifndef ORACLE_STORAGE_FORMATS_H
#define ORACLE_STORAGE_FORMATS_H

#include <stdint.h>
#include <string.h>

enum { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2 };

/* ------------------------------------------------------------------------ */
/* storage formats                                                          */
/* ------------------------------------------------------------------------ */
static inline float u32_as_float(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t float_as_u32(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bf16_to_float(uint16_t h) { return u32_as_float((uint32_t)h << 16); }

static inline uint16_t float_to_bf16(float f)
{
    uint32_t u = float_as_u32(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u);                                             /* nearest even */
    return (uint16_t)(u >> 16);
}

static inline float f16_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    const uint32_t man = h & 0x3ffu;
    if (exp == 0x1fu) return u32_as_float(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        /* zero or subnormal: man * 2^-24, exact in fp32 */
        const float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return u32_as_float(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t float_to_f16(float f)
{
    const uint32_t u = float_as_u32(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return sign;                        /* <= 2^-25 rounds to zero */
    const int e = (int)(a >> 23) - 127;
    uint32_t man = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;                                  /* bits dropped from the significand */
    uint32_t base;
    if (e < -14) {
        shift = 13 + (-14 - e); /* subnormal result */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    const uint32_t kept = man >> shift;
    const uint32_t rest = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t r = base + kept; /* a carry out of the mantissa bumps the exponent, as it should */
    if (rest > half || (rest == half && (kept & 1u))) r += 1;
    return (uint16_t)(sign | r);
}

static inline float load_elem(const void* p, int64_t i, int dt)
{
    if (dt == DT_BF16) return bf16_to_float(((const uint16_t*)p)[i]);
    if (dt == DT_F16) return f16_to_float(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}
static inline void store_elem(void* p, int64_t i, int dt, float v)
{
    if (dt == DT_BF16)
        ((uint16_t*)p)[i] = float_to_bf16(v);
    else if (dt == DT_F16)
        ((uint16_t*)p)[i] = float_to_f16(v);
    else
        ((float*)p)[i] = v;
}
/* value of v after a round trip through storage type dt */
static inline float round_to(float v, int dt)
{
    if (dt == DT_BF16) return bf16_to_float(float_to_bf16(v));
    if (dt == DT_F16) return f16_to_float(float_to_f16(v));
    return v;
}

/* a (*) b and a (+) b of the 16-bit scalar types (c10::Half / c10::BFloat16 operators, and torch's eager
 * kernels for these dtypes): the fp32 operation, then rounding to the storage type
 * (fused_rotary_positional_embedding.h:58,107,158,209 use scalar_t operators). */
static inline float mul_t(float a, float b, int dt) { return round_to(a * b, dt); }
static inline float add_t(float a, float b, int dt) { return round_to(a + b, dt); }

static inline float pairwise_sum(const float* v, int64_t n)
{
    if (n <= 8) {
        float s = 0.0f;
        for (int64_t i = 0; i < n; ++i) s += v[i];
        return s;
    }
    const int64_t h = n / 2;
    return pairwise_sum(v, h) + pairwise_sum(v + h, n - h);
}


#endif
