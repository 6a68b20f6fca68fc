// Small device helpers shared by the gfx950 kernels: vector typedefs, bf16 packing, exp2, the replay-parameter
// resolver and the sigmoid used by the gate (gqa_activation_gate.metal:14-26 of the reference).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_params.h"

namespace khm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4v __attribute__((ext_vector_type(4)));

// LDS transpose read: lane r of every 16-lane group passes the address of 4 consecutive bf16; lane i receives
// element (i % 4) of the rows given by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 of its group.
__device__ __forceinline__ s16x4v lds_read_tr16(const unsigned char* address) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4v __attribute__((address_space(3)))*)(address));
}

__device__ __forceinline__ uint32_t resolve_u32(DeviceReplayU32 r, const uint32_t* params) {
    return r.is_parameter ? params[r.value] : r.value;
}

// A word of a table that does not change while the kernel runs, read with a wave-uniform index through the constant
// address space: the compiler then issues a scalar load (its own counter) instead of a vector load, and consecutive ones
// with no branch between them go out together and are waited for once.
__device__ __forceinline__ uint32_t load_uniform_u32(const uint32_t* table, uint64_t index) {
    typedef const uint32_t __attribute__((address_space(4))) * ConstantU32;
    return ((ConstantU32)(uintptr_t)table)[index];
}

// Makes the kernel read its whole argument block when it starts.  Left alone, the compiler fetches each group of
// arguments where it is first used, behind the branches of the task decode: two more dependent round trips to memory in
// front of a block's first K/V load.
__device__ __forceinline__ void fetch_all_arguments(const MapParams& p) {
    asm volatile("" ::"s"(p.q), "s"(p.kv_pages), "s"(p.req_slots), "s"(p.page_ids), "s"(p.visible_ranges), "s"(p.q_token_ranges),
                 "s"(p.templates), "s"(p.exp_sums), "s"(p.max_logits), "s"(p.out), "s"(p.replay_parameters));
    asm volatile("" ::"s"(p.page_bytes), "s"(p.num_q_heads), "s"(p.num_kv_heads), "s"(p.q_heads_per_kv_head), "s"(p.max_q_heads),
                 "s"(p.num_q_head_ranges), "s"(p.max_q_tokens), "s"(p.tokens_per_page), "s"(p.tokens_per_page_shift),
                 "s"(p.num_gqa_layers), "s"(p.pages_per_request_layer), "s"(p.output_mode), "s"(p.scale_log2e));
}

// The four replay values of a Map launch, each fixed or read from the parameter block; the reads are issued together.
struct ReplayValues {
    uint32_t layer, num_active_tokens, num_active_q_token_tiles, num_active_kv_splits;
};
__device__ __forceinline__ ReplayValues resolve_replay_values(const MapParams& p) {
    // with no parameter block every value is fixed and the words read here (any readable ones) are not used
    const uint32_t* source = p.replay_parameters != nullptr ? p.replay_parameters : p.templates;
    const uint32_t a = load_uniform_u32(source, p.layer_index.is_parameter ? p.layer_index.value : 0u);
    const uint32_t b = load_uniform_u32(source, p.num_active_tokens.is_parameter ? p.num_active_tokens.value : 0u);
    const uint32_t c = load_uniform_u32(source, p.num_active_q_token_tiles.is_parameter ? p.num_active_q_token_tiles.value : 0u);
    const uint32_t d = load_uniform_u32(source, p.num_active_kv_splits.is_parameter ? p.num_active_kv_splits.value : 0u);
    return ReplayValues{p.layer_index.is_parameter ? a : p.layer_index.value,
                        p.num_active_tokens.is_parameter ? b : p.num_active_tokens.value,
                        p.num_active_q_token_tiles.is_parameter ? c : p.num_active_q_token_tiles.value,
                        p.num_active_kv_splits.is_parameter ? d : p.num_active_kv_splits.value};
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// e^x through v_exp_f32; both Reduce implementations use this one so they agree bit for bit.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

// Combining one value per 16-lane row over the four rows of a wave (lanes l, l^16, l^32, l^48), result in every lane.
// gfx950 swaps lane rows inside the VALU (v_permlane16_swap / v_permlane32_swap); a generic shuffle would go through
// the LDS crossbar, whose result also queues behind every LDS read in flight.
__device__ __forceinline__ float max_over_rows(float x) {
    uint32_t bits = __float_as_uint(x);
    auto halves = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    bits = __float_as_uint(fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1])));
    halves = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    return fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
}
__device__ __forceinline__ float sum_over_rows(float x) {
    uint32_t bits = __float_as_uint(x);
    auto halves = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    bits = __float_as_uint(__uint_as_float(halves[0]) + __uint_as_float(halves[1]));
    halves = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    return __uint_as_float(halves[0]) + __uint_as_float(halves[1]);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// Streaming accesses (the nt bit of the memory instruction: a hint that the bytes will not be used again soon), for bytes
// that are written once for a later launch, or read once by this block and by no other.  Measured: decode Map 107 -> 98 us
// on a 32-request batch and verify tiles 240 -> 223 us with streaming K/V loads, at unchanged HBM traffic; RMSNorm + RoPE
// rows 102 -> 86 us with streaming stores (94 us with streaming loads as well, so its loads stay ordinary ones); K/V tiles
// that several blocks share through the L2 (prefill) lose with the hint and do not get it.
__device__ __forceinline__ void store_streaming(void* target, uint4 value) {
    typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
    const U32x4 v = {value.x, value.y, value.z, value.w};
    __builtin_nontemporal_store(v, reinterpret_cast<U32x4*>(target));
}
__device__ __forceinline__ void store_streaming(void* target, uint2 value) {
    typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));
    const U32x2 v = {value.x, value.y};
    __builtin_nontemporal_store(v, reinterpret_cast<U32x2*>(target));
}
__device__ __forceinline__ void store_streaming(void* target, float4 value) {
    typedef float F32x4 __attribute__((ext_vector_type(4)));
    const F32x4 v = {value.x, value.y, value.z, value.w};
    __builtin_nontemporal_store(v, reinterpret_cast<F32x4*>(target));
}
__device__ __forceinline__ uint4 load_streaming(const void* source) {
    typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
    const U32x4 v = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(source));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) { return __uint_as_float(bits << 16); }

// Round-to-nearest-even f32 -> bf16 bits (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) { return (uint16_t)(pack_bf16x2(v, 0.0f) & 0xffffu); }

// Device-coherent accesses for data that another block on another XCD produces or consumes within one kernel:
// relaxed agent-scope atomics compile to sc1 loads/stores that are served by memory instead of this XCD's
// L2, so no cache write-back or invalidate is needed around them.
__device__ __forceinline__ void coherent_store_u64(void* address, uint64_t value) {
    __hip_atomic_store(reinterpret_cast<uint64_t*>(address), value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coherent_store_f32(float* address, float value) {
    __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t coherent_load_u64(const void* address) {
    return __hip_atomic_load(reinterpret_cast<const uint64_t*>(address), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load_f32(const float* address) {
    return __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float round_to_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// gqa_activation_gate.metal:19-26: sigmoid with every step rounded to bf16.
// `x` is a decoded bf16 value (every caller passes one), so |x| and -|x| are bf16 values already and their rounding steps
// are identities; the denominator is one of the 129 bf16 values in [1, 2], for each of which v_rcp_f32 rounds to the same
// bf16 as the exact quotient (checked, with everything else, over all 65 536 gate patterns against the oracle).
__device__ __forceinline__ float sigmoid_bf16_steps(float x) {
    const float neg_abs_x = -fabsf(x);
    const float exp_x = round_to_bf16(__expf(neg_abs_x));
    const float denom = round_to_bf16(1.0f + exp_x);
    const float y = round_to_bf16(__builtin_amdgcn_rcpf(denom));
    return x < 0.0f ? round_to_bf16(1.0f - y) : y;
}

// Four attention values times sigmoid(gate) as gqa_activation_gate_bf16 computes it from the bf16-rounded attention
// output (gqa_activation_gate.metal:19-39); `gates` points at the four bf16 gate values of the same elements.
__device__ __forceinline__ f32x4 gate_bf16x4(f32x4 attention, const uint16_t* gates) {
    const uint2 gate_bits = *reinterpret_cast<const uint2*>(gates);
    const float gate[4] = {bf16_bits_to_f32(gate_bits.x & 0xffffu), bf16_bits_to_f32(gate_bits.x >> 16),
                           bf16_bits_to_f32(gate_bits.y & 0xffffu), bf16_bits_to_f32(gate_bits.y >> 16)};
#pragma unroll
    for (int i = 0; i < 4; ++i) attention[i] = round_to_bf16(attention[i]) * sigmoid_bf16_steps(gate[i]);
    return attention;
}

// gqa_activation_gate.metal:14-17.
__device__ __forceinline__ float sigmoid_f32(float x) {
    const float y = 1.0f / (1.0f + __expf(-fabsf(x)));
    return x < 0.0f ? 1.0f - y : y;
}

}  // namespace khm
