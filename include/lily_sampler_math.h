/*
 * lily_sampler_math.h - the exact scalar arithmetic of the logits-to-token stage.
 *
 * Everything here is plain IEEE-754 binary32 / 64-bit integer arithmetic with no
 * fused operations, so the same source gives the same bits under gcc on the
 * host and under hipcc on gfx950 (both built with -ffp-contract=off, default
 * rounding, denormals kept).  The HIP kernels and any host code that wants to
 * replay a draw include this header.
 *
 *   lilym_uniform_for  - the (seed, step) -> [0,1) draw.
 *       Replaces: src/kernels/sample.rs:435-441 (uniform_for) and
 *                 src/kernels/metal/sample.metal:93-101 (sample_uniform).
 *   lilym_draft_step / lilym_residual_step - RNG index domains.
 *       Replaces: src/kernels/sample.rs:220-222 (draft_step),
 *                 src/kernels/metal/sample.metal:649 (step | 0x80000000).
 *   lilym_order_key    - monotone float -> uint key (f32::total_cmp order).
 *       Replaces: src/kernels/metal/sample.metal:29-32 (sample_key).
 *   lilym_expf         - the exp() of the candidate softmax.
 *       Replaces: f32::exp at tests/unit/kernels/sample.rs:37 and `exp` at
 *       src/kernels/metal/sample.metal:419.  The reference takes the
 *       platform's libm here, whose bits are not portable; this build fixes
 *       one software implementation (Cody-Waite reduction, degree-6
 *       polynomial, about 1 ulp) so that host replay and device agree
 *       bit for bit.
 */
#ifndef LILY_SAMPLER_MATH_H
#define LILY_SAMPLER_MATH_H

#include <stdint.h>

#if defined(__HIPCC__)
#define LILY_HD __host__ __device__ static inline
#else
#define LILY_HD static inline
#endif

LILY_HD uint32_t lilym_f32_bits(float x) {
    uint32_t u;
    __builtin_memcpy(&u, &x, 4);
    return u;
}

LILY_HD float lilym_bits_f32(uint32_t u) {
    float x;
    __builtin_memcpy(&x, &u, 4);
    return x;
}

/* Greater floats give greater keys; the order is f32::total_cmp's
 * (-NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN). */
LILY_HD uint32_t lilym_order_key(float v) {
    const uint32_t u = lilym_f32_bits(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

LILY_HD float lilym_key_value(uint32_t key) {
    return lilym_bits_f32((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

/* bf16 -> f32 is exact: the 16 stored bits are the top half of the f32. */
LILY_HD float lilym_bf16_to_f32(uint16_t h) {
    return lilym_bits_f32((uint32_t)h << 16);
}

/* SplitMix64 finaliser of seed + step * golden; top 24 bits scaled to [0,1). */
LILY_HD float lilym_uniform_for(uint64_t seed, uint32_t step) {
    uint64_t z = seed + (uint64_t)step * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(uint32_t)(z >> 40) * (1.0f / 16777216.0f);
}

LILY_HD uint32_t lilym_draft_step(uint32_t step) { return step | 0x40000000u; }
LILY_HD uint32_t lilym_residual_step(uint32_t step) { return step | 0x80000000u; }

/* exp(x) in binary32.  n = round(x/ln2); r = x - n*ln2 in two exact-ish
 * steps (the high part of ln2 has 9 trailing zero bits, so n*hi is exact for
 * |n| < 512); e^r by a degree-6 polynomial on |r| <= 0.3466; the result is
 * scaled by 2^n in two power-of-two multiplications so that a subnormal
 * result is rounded once. */
LILY_HD float lilym_expf(float x) {
    if (x != x) {
        return x;
    }
    if (x > 88.72283935546875f) {
        return lilym_bits_f32(0x7f800000u);
    }
    if (x < -103.97208404541015625f) {
        return 0.0f;
    }
    const float t = x * 1.44269502162933349609375f;
    const float n = (t + 12582912.0f) - 12582912.0f;
    float r = x - n * 0.693145751953125f;
    r = r - n * 1.428606765330187045e-06f;
    const float r2 = r * r;
    float p = 1.9875691500e-4f;
    p = p * r + 1.3981999507e-3f;
    p = p * r + 8.3334519073e-3f;
    p = p * r + 4.1665795894e-2f;
    p = p * r + 1.6666665459e-1f;
    p = p * r + 5.0000001201e-1f;
    float y = p * r2 + r;
    y = y + 1.0f;
    const int ni = (int)n;
    const int h = ni >> 1;
    const float s1 = lilym_bits_f32((uint32_t)(h + 127) << 23);
    const float s2 = lilym_bits_f32((uint32_t)(ni - h + 127) << 23);
    y = y * s1;
    return y * s2;
}

#endif /* LILY_SAMPLER_MATH_H */
