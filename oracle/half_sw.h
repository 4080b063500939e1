/*
 * Software float16 <-> float32 conversions shared by the oracle's C files -- TEST
 * INFRASTRUCTURE ONLY (never linked into the product library).
 */
#ifndef ORACLE_HALF_SW_H
#define ORACLE_HALF_SW_H
#include <stdint.h>
#include <string.h>

/* ---- software float16 <-> float32 (round to nearest even) ------------------------------
 * Semantics of include/hidet/runtime/cpu/float16.h:132-393: IEEE binary16, RNE, subnormals
 * kept.  Written from the format definition, not from that file. */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static inline uint16_t half_from_f32(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) return (uint16_t)(sign | (ax > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf */
    if (ax < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 rounds to 0 */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7FFFFFu) | 0x800000u;
    uint32_t shift, half_bits;
    if (e < -14) {            /* subnormal half: value = man * 2^(e-23), unit 2^-24 */
        shift = (uint32_t)(-1 - e);      /* 13 + (-14 - e) */
        half_bits = 0;
    } else {
        shift = 13;
        half_bits = (uint32_t)(e + 15) << 10;
        man &= 0x7FFFFFu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    uint32_t r = half_bits + q;
    if (rem > halfway || (rem == halfway && (q & 1u))) r += 1; /* carries into exponent correctly */
    return (uint16_t)(sign | r);
}

static inline float half_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0x1F) return bits_f32(sign | 0x7F800000u | (m << 13));
    if (e == 0) {
        float v = (float)m * 5.9604644775390625e-8f; /* m * 2^-24, exact */
        return sign ? -v : v;
    }
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

#endif
