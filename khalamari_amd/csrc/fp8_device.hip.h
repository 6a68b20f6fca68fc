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

// Two bf16 bit patterns (low and high half of `pair`) to their two E4M3FN codes (bits 0..7 and 8..15) through the
// hardware converter v_cvt_pk_fp8_f32 (round to nearest even, subnormals below 2^-6).  The converter does not
// saturate by itself, so finite and infinite magnitudes are clamped to 448 first; NaN keeps its sign and becomes 0x7f.
// Checked against the integer encoder above and the host codec over all 65 536 patterns in both positions.
__device__ __forceinline__ uint32_t bf16x2_bits_to_fp8x2_e4m3fn(uint32_t pair) {
    const float low = __uint_as_float(pair << 16), high = __uint_as_float(pair & 0xffff0000u);
    const float low_clamped = __builtin_amdgcn_fmed3f(low, -448.0f, 448.0f);
    const float high_clamped = __builtin_amdgcn_fmed3f(high, -448.0f, 448.0f);
    uint32_t codes = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(low_clamped, high_clamped, 0, false) & 0xffffu;
    if ((pair & 0x7fffu) > 0x7f80u) codes = (codes & 0xff00u) | ((pair >> 8) & 0x80u) | 0x7fu;
    if ((pair & 0x7fff0000u) > 0x7f800000u) codes = (codes & 0x00ffu) | ((pair >> 16) & 0x8000u) | 0x7f00u;
    return codes;
}

}  // namespace khm
