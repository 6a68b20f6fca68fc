// Log-sum-exp merge of split-KV partial states, shared by the Reduce kernels and the fused Map epilogue.
//
// Contract of the reference's reducers (gqa_sdpa_sliced_kv_reduce.metal:30-55, gqa_sdpa_sliced_q_reduce.metal:27-62):
//     w_p = exp(max_p - gmax) * sum_p, 0 for an empty partial;  out = sum_p w_p * partial_p / sum_p w_p.
// Here the walk over partials is a single online pass (running max, rescale on increase) so that the loads of
// eight partials can be in flight at once instead of one dependent load per step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.hip.h"

namespace khm {

struct MergeState {
    float run_max;
    float run_sum;
    f32x4 acc;
};

__device__ __forceinline__ MergeState merge_state_empty() { return MergeState{-INFINITY, 0.0f, f32x4{0.0f, 0.0f, 0.0f, 0.0f}}; }

template <bool COHERENT>
__device__ __forceinline__ float merge_load_f32(const float* address) {
    if constexpr (COHERENT) return coherent_load_f32(address);
    return *address;
}

template <bool COHERENT>
__device__ __forceinline__ uint64_t merge_load_u64(const void* address) {
    if constexpr (COHERENT) return coherent_load_u64(address);
    return *reinterpret_cast<const uint64_t*>(address);
}

// Merges partials first, first + step, ... < end of one (Q head, token offset) row into `state`, for the four
// dims chunk*4 .. chunk*4+3.  `safe_part` is any valid partial index (address of masked-off batch slots).
template <int D, bool COHERENT, int BATCH = 8>
__device__ __forceinline__ void merge_partial_slice(MergeState& state, const float* max_logits, const float* exp_sums, const void* partial,
                                                    bool f32_partials, uint32_t first, uint32_t end, uint32_t step, uint32_t safe_part,
                                                    uint32_t num_q_heads, uint32_t q_head, uint32_t max_q_tokens, uint32_t token_offset,
                                                    int chunk) {
    for (; first < end; first += BATCH * step) {
        float part_max[BATCH], part_sum[BATCH];
        uint64_t lo[BATCH], hi[BATCH];
#pragma unroll
        for (int k = 0; k < BATCH; ++k) {
            const uint32_t part = first + k * step;
            const bool ok = part < end;
            const uint64_t row = ((uint64_t)(ok ? part : safe_part) * num_q_heads + q_head) * max_q_tokens + token_offset;
            part_max[k] = merge_load_f32<COHERENT>(max_logits + row);
            part_sum[k] = ok ? merge_load_f32<COHERENT>(exp_sums + row) : 0.0f;
            if (f32_partials) {
                const float* source = reinterpret_cast<const float*>(partial) + row * D + chunk * 4;
                lo[k] = merge_load_u64<COHERENT>(source);
                hi[k] = merge_load_u64<COHERENT>(source + 2);
            } else {
                lo[k] = merge_load_u64<COHERENT>(reinterpret_cast<const uint16_t*>(partial) + row * D + chunk * 4);
                hi[k] = 0;
            }
        }
#pragma unroll
        for (int k = 0; k < BATCH; ++k) {
            if (!(part_sum[k] > 0.0f) || !(fabsf(part_max[k]) < INFINITY)) continue;  // empty partial
            f32x4 value;
            if (f32_partials) {
                value = f32x4{__uint_as_float((uint32_t)lo[k]), __uint_as_float((uint32_t)(lo[k] >> 32)),
                              __uint_as_float((uint32_t)hi[k]), __uint_as_float((uint32_t)(hi[k] >> 32))};
            } else {
                const uint32_t a = (uint32_t)lo[k], b = (uint32_t)(lo[k] >> 32);
                value = f32x4{bf16_bits_to_f32(a & 0xffffu), bf16_bits_to_f32(a >> 16), bf16_bits_to_f32(b & 0xffffu), bf16_bits_to_f32(b >> 16)};
            }
            const float next_max = fmaxf(state.run_max, part_max[k]);
            const float keep = fast_exp(state.run_max - next_max);  // 0 while run_max is still -inf
            const float weight = fast_exp(part_max[k] - next_max) * part_sum[k];
            state.run_sum = state.run_sum * keep + weight;
            state.acc = state.acc * keep + value * weight;
            state.run_max = next_max;
        }
    }
}

// Combines `count` slice states stored in LDS (stats [i][2] = (max, sum), acc [i][D]) for this lane's chunk.
template <int D>
__device__ __forceinline__ MergeState merge_combine_slices(const float* stats, const float* acc, uint32_t first, uint32_t count, int chunk) {
    float all_max = -INFINITY;
    for (uint32_t i = 0; i < count; ++i) all_max = fmaxf(all_max, stats[(first + i) * 2]);
    MergeState out = merge_state_empty();
    out.run_max = all_max;
    for (uint32_t i = 0; i < count; ++i) {
        const float slice_sum = stats[(first + i) * 2 + 1];
        if (slice_sum > 0.0f) {
            const float factor = fast_exp(stats[(first + i) * 2] - all_max);
            out.run_sum += slice_sum * factor;
            out.acc += *reinterpret_cast<const f32x4*>(acc + (first + i) * D + chunk * 4) * factor;
        }
    }
    return out;
}

// Normalizes, applies the optional bf16 gate (gqa_activation_gate.metal:19-39) and stores four bf16 outputs.
__device__ __forceinline__ void merge_store_output(const MergeState& state, uint16_t* output, const uint16_t* gates, uint64_t out_index) {
    f32x4 result = {0.0f, 0.0f, 0.0f, 0.0f};
    if (state.run_sum > 0.0f) result = state.acc / state.run_sum;
    if (gates != nullptr) result = gate_bf16x4(result, gates + out_index);
    const uint2 packed = make_uint2(pack_bf16x2(result[0], result[1]), pack_bf16x2(result[2], result[3]));
    *reinterpret_cast<uint2*>(output + out_index) = packed;
}

}  // namespace khm
