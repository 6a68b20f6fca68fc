// Host-side FP8 E4M3FN unit-scale codec used for GQA K/V pages.  Contract of
// crates/inference-backend-metal/src/components/gqa/fp8.rs:19-58: round to nearest even,
// finite and infinite inputs saturate to +/-448 (0x7e / 0xfe), NaN maps to 0x7f / 0xff.
// Implemented on the bf16 bit pattern directly (integer arithmetic only) instead of the reference's
// log2/floor formulation; both are exact, so the 65536-entry encode table is identical.
#include "common.h"

extern "C" uint16_t khm_f32_to_bf16(float value) {
    uint32_t bits;
    __builtin_memcpy(&bits, &value, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x0040u);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

extern "C" float khm_bf16_to_f32(uint16_t bf16_bits) {
    const uint32_t bits = (uint32_t)bf16_bits << 16;
    float value;
    __builtin_memcpy(&value, &bits, 4);
    return value;
}

extern "C" uint8_t khm_bf16_to_fp8_e4m3(uint16_t bf16_bits) {
    const uint8_t sign = (bf16_bits & 0x8000u) ? 0x80 : 0x00;
    const uint32_t magnitude = bf16_bits & 0x7fffu;
    const uint32_t exponent = magnitude >> 7;  // biased by 127
    const uint32_t mantissa = magnitude & 0x7fu;
    if (exponent == 0xff) return sign | (mantissa ? 0x7f : 0x7e);
    // bf16 value = (128 + mantissa) * 2^(exponent - 134) for normals.
    if (exponent >= 127 + 9) return sign | 0x7e;  // >= 512
    if (exponent < 127 - 6) {
        // E4M3 subnormal grid: multiples of 2^-9.  q = round_ties_even(value * 512).
        if (exponent == 0) return sign;  // bf16 subnormals are far below 2^-10
        const int shift = (int)(134 - 9) - (int)exponent;  // value * 512 = (128 + m) >> shift
        if (shift > 9) return sign;
        const uint32_t significand = 128u + mantissa;
        const uint32_t floor_q = significand >> shift;
        const uint32_t remainder = significand & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1);
        uint32_t q = floor_q;
        if (remainder > half || (remainder == half && (floor_q & 1u))) q += 1;
        return sign | (uint8_t)(q < 8 ? q : 8);
    }
    // Normal range: keep 3 mantissa bits of the 7, ties to even, carry into the exponent.
    uint32_t kept = mantissa >> 4;
    const uint32_t dropped = mantissa & 0xfu;
    uint32_t e4 = exponent - 127 + 7;
    if (dropped > 8 || (dropped == 8 && (kept & 1u))) kept += 1;
    if (kept == 8) {
        kept = 0;
        e4 += 1;
    }
    if (e4 > 15 || (e4 == 15 && kept >= 7)) return sign | 0x7e;
    return sign | (uint8_t)(e4 << 3) | (uint8_t)kept;
}

extern "C" uint16_t khm_fp8_e4m3_to_bf16(uint8_t fp8_bits) {
    const uint16_t sign = (fp8_bits & 0x80) ? 0x8000 : 0;
    const uint32_t exponent = (fp8_bits >> 3) & 0x0f;
    const uint32_t mantissa = fp8_bits & 0x07;
    if (exponent == 15 && mantissa == 7) return sign | 0x7fc0;
    if (exponent == 0) {
        if (mantissa == 0) return sign;
        // mantissa * 2^-9, normalised: the leading bit of the 3-bit mantissa sets the exponent.
        const int top = 31 - __builtin_clz(mantissa);
        const uint32_t bf16_exponent = 127 - 9 + top;
        const uint32_t bf16_mantissa = ((mantissa << (7 - top)) & 0x7fu);
        return sign | (uint16_t)(bf16_exponent << 7) | (uint16_t)bf16_mantissa;
    }
    return sign | (uint16_t)((exponent + 120) << 7) | (uint16_t)(mantissa << 4);
}
