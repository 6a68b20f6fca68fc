// FP8 E4M3FN unit-scale codec on the device (gfx950).
//
// Decode replaces fp8_e4m3x8_to_bf16x8 of the reference's shaders (crates/inference-backend-metal/src/components/
// metal/gqa_fp8.metal:1-25); encode replaces bf16_to_fp8_e4m3 of the page writer (.../metal/gqa_kv_page_write.metal:5-31,
// components/gqa/fp8.rs:19-45): round to nearest even, finite and infinite inputs saturate to +/-448 (0x7e), NaN keeps
// the E4M3FN NaN code (0x7f).  Every E4M3FN value is exactly representable in bf16, so decoding is exact.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.hip.h"

namespace khm {

// Two E4M3FN codes (the low or the high half of `codes`) to two bf16 values in one 32-bit word.  gfx950 converts OCP
// FP8 in hardware; the scale operand is a power of two and 1.0 leaves the value unchanged.
template <bool HIGH_HALF>
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t codes) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(codes, 1.0f, HIGH_HALF));
}

// Eight codes (two words) to eight bf16 (four words), element order preserved.
__device__ __forceinline__ uint4 fp8x8_to_bf16x8(uint2 codes) {
    return make_uint4(fp8x2_to_bf16x2<false>(codes.x), fp8x2_to_bf16x2<true>(codes.x), fp8x2_to_bf16x2<false>(codes.y),
                      fp8x2_to_bf16x2<true>(codes.y));
}

// One bf16 bit pattern to its E4M3FN code, in integer arithmetic on the bf16 fields (7-bit mantissa -> 3 bits).
__device__ __forceinline__ uint32_t bf16_bits_to_fp8_e4m3fn(uint32_t bits) {
    const uint32_t sign = (bits >> 8) & 0x80u;
    const uint32_t magnitude = bits & 0x7fffu;
    if (magnitude > 0x7f80u) return sign | 0x7fu;             // NaN
    if (magnitude >= 0x43e0u) return sign | 0x7eu;            // >= 448 or infinite: saturate
    const uint32_t exponent = magnitude >> 7;                 // biased by 127
    if (exponent < 121u) {                                    // below 2^-6: E4M3FN subnormal, step 2^-9
        const float scaled = __uint_as_float(magnitude << 16) * 512.0f;
        const uint32_t mantissa = (uint32_t)__builtin_rintf(scaled);   // round half to even
        return sign | (mantissa < 8u ? mantissa : 8u);
    }
    uint32_t kept = (magnitude >> 4) & 0x7u;
    const uint32_t dropped = magnitude & 0xfu;
    uint32_t encoded_exponent = exponent - 120u;              // (exponent - 127) + 7
    if (dropped > 8u || (dropped == 8u && (kept & 1u))) ++kept;
    if (kept == 8u) {
        kept = 0u;
        ++encoded_exponent;
    }
    if (encoded_exponent > 15u || (encoded_exponent == 15u && kept >= 7u)) return sign | 0x7eu;
    return sign | (encoded_exponent << 3) | kept;
}

// Two bf16 bit patterns (low and high half of `pair`) to their two E4M3FN codes, written to the low (HIGH_HALF = false)
// or high 16 bits of `old` through v_cvt_scalef32_pk_fp8_bf16 with scale 1 (round to nearest even, subnormals below
// 2^-6).  The converter does not saturate (magnitudes above 464 come out as the NaN code), so magnitudes are clamped to
// 448 first, as 16-bit integers on the bf16 fields, which orders finite and infinite magnitudes alike; NaN would be
// clamped with them and is patched afterwards: it keeps its sign and becomes 0x7f.  Checked against the integer encoder
// above and the host codec over all 65 536 patterns in every position.
typedef unsigned short Fp8U16x2 __attribute__((ext_vector_type(2)));
typedef short Fp8I16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 Fp8Bf16x2 __attribute__((ext_vector_type(2)));

template <bool HIGH_HALF>
__device__ __forceinline__ uint32_t bf16x2_bits_to_fp8x2_no_nan(uint32_t old, uint32_t pair) {
    const Fp8U16x2 magnitude = __builtin_bit_cast(Fp8U16x2, pair & 0x7fff7fffu);
    const Fp8U16x2 limit = {0x43e0, 0x43e0};
    const uint32_t clamped = (pair & 0x80008000u) | __builtin_bit_cast(uint32_t, __builtin_elementwise_min(magnitude, limit));
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(__builtin_bit_cast(Fp8I16x2, old),
                                                                                 __builtin_bit_cast(Fp8Bf16x2, clamped), 1.0f, HIGH_HALF));
}

// Nonzero in the half of the result whose half of `pair` is a NaN.
__device__ __forceinline__ uint32_t bf16x2_nan_halves(uint32_t pair) {
    const Fp8U16x2 magnitude = __builtin_bit_cast(Fp8U16x2, pair & 0x7fff7fffu);
    const Fp8U16x2 infinity = {0x7f80, 0x7f80};
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_sub_sat(magnitude, infinity));
}

__device__ __forceinline__ uint32_t bf16x2_bits_to_fp8x2_e4m3fn(uint32_t pair) {
    uint32_t codes = bf16x2_bits_to_fp8x2_no_nan<false>(0u, pair) & 0xffffu;
    const uint32_t nan = bf16x2_nan_halves(pair);
    if (nan != 0u) {
        if ((nan & 0xffffu) != 0u) codes = (codes & 0xff00u) | ((pair >> 8) & 0x80u) | 0x7fu;
        if ((nan >> 16) != 0u) codes = (codes & 0x00ffu) | ((pair >> 16) & 0x8000u) | 0x7f00u;
    }
    return codes;
}

// Four bf16 bit patterns (`first` holds elements 0 and 1, `second` elements 2 and 3) to four codes in element order.
__device__ __forceinline__ uint32_t bf16x4_bits_to_fp8x4_e4m3fn(uint32_t first, uint32_t second) {
    uint32_t codes = bf16x2_bits_to_fp8x2_no_nan<true>(bf16x2_bits_to_fp8x2_no_nan<false>(0u, first), second);
    const uint32_t nan_first = bf16x2_nan_halves(first), nan_second = bf16x2_nan_halves(second);
    if ((nan_first | nan_second) != 0u) {
        if ((nan_first & 0xffffu) != 0u) codes = (codes & 0xffffff00u) | ((first >> 8) & 0x80u) | 0x7fu;
        if ((nan_first >> 16) != 0u) codes = (codes & 0xffff00ffu) | ((first >> 16) & 0x8000u) | 0x7f00u;
        if ((nan_second & 0xffffu) != 0u) codes = (codes & 0xff00ffffu) | ((second << 8) & 0x800000u) | 0x7f0000u;
        if ((nan_second >> 16) != 0u) codes = (codes & 0x00ffffffu) | (second & 0x80000000u) | 0x7f000000u;
    }
    return codes;
}

// Eight bf16 bit patterns to eight codes, element order preserved.
__device__ __forceinline__ uint2 bf16x8_bits_to_fp8x8_e4m3fn(uint4 bits) {
    return make_uint2(bf16x4_bits_to_fp8x4_e4m3fn(bits.x, bits.y), bf16x4_bits_to_fp8x4_e4m3fn(bits.z, bits.w));
}

}  // namespace khm
