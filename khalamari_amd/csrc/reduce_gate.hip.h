// Log-sum-exp Reduce kernels and the sigmoid gate for gfx950.
//
// split_kv_reduce_kernel replaces gqa_sdpa_sliced_kv_reduce_bf16
// (crates/inference-backend-metal/src/components/metal/gqa_sdpa_sliced_kv_reduce.metal:10-56) and
// gqa_sdpa_sliced_q_reduce (.../gqa_sdpa_sliced_q_reduce.metal:4-63):
//     gmax = max_p max_p;  w_p = exp(max_p - gmax) * sum_p  (0 for an empty partial);
//     out  = sum_p w_p * partial_p / sum_p w_p              (0 when the denominator is 0)
// One block owns one output row group; its threads are arranged as
// (partial-slice, 4-dim chunk): every slice walks a strided subset of the row's partials with
// its own running maximum, and the slices are merged through LDS.  Long rows (a 131072-token
// context has 64 partials at 2048-token partitions) therefore reduce in parallel instead of in
// one thread's serial loop.
//
// The optional gate epilogue is gqa_activation_gate_bf16 (.../gqa_activation_gate.metal:19-39)
// applied to the bf16-rounded attention value, which is what the reference's separate kernel sees.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_params.h"
#include "split_kv_map.hip.h"

namespace khm {

__device__ __forceinline__ float round_to_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// gqa_activation_gate.metal:19-26: sigmoid with every step rounded to bf16.
__device__ __forceinline__ float sigmoid_bf16_steps(float x) {
    const float abs_x = round_to_bf16(fabsf(x));
    const float neg_abs_x = round_to_bf16(-abs_x);
    const float exp_x = round_to_bf16(__expf(neg_abs_x));
    const float denom = round_to_bf16(1.0f + exp_x);
    const float y = round_to_bf16(1.0f / denom);
    return x < 0.0f ? round_to_bf16(1.0f - y) : y;
}

// gqa_activation_gate.metal:14-17.
__device__ __forceinline__ float sigmoid_f32(float x) {
    const float y = 1.0f / (1.0f + __expf(-fabsf(x)));
    return x < 0.0f ? 1.0f - y : y;
}

constexpr int kReduceThreads = 256;

// RANGED = false: sliced-KV flat reduce, grid (tokens, heads).
// RANGED = true : sliced-Q reduce, grid (Q ranges, heads); loops the range's tokens.
template <int D, bool RANGED>
__global__ __launch_bounds__(kReduceThreads) void split_kv_reduce_kernel(const ReduceParams p) {
    constexpr int CHUNKS = D / 4;                    // threads per row
    constexpr int SLICES = kReduceThreads / CHUNKS;  // partial slices per block
    __shared__ float slice_max[SLICES];
    __shared__ float slice_sum[SLICES];
    __shared__ __align__(16) float slice_acc[SLICES][D];

    const uint32_t unit = blockIdx.x;
    if (unit >= resolve_u32(p.num_active, p.replay_parameters)) return;
    const uint32_t head = blockIdx.y;
    const uint32_t begin = p.cu_partial_outputs[unit];
    const uint32_t end = p.cu_partial_outputs[unit + 1];
    uint32_t flat_begin = unit, num_q = 1, max_q = 1;
    if (RANGED) {
        flat_begin = p.q_token_ranges[2 * (uint64_t)unit];
        num_q = p.q_token_ranges[2 * (uint64_t)unit + 1] - flat_begin;
        max_q = p.max_q_tokens;
        if (num_q > max_q) num_q = max_q;
    }
    const int chunk = threadIdx.x % CHUNKS;
    const int slice = threadIdx.x / CHUNKS;

    for (uint32_t local = 0; local < num_q; ++local) {
        float local_max = -INFINITY;
        for (uint32_t part = begin + slice; part < end; part += SLICES) {
            const uint64_t state = ((uint64_t)part * p.num_q_heads + head) * max_q + local;
            local_max = fmaxf(local_max, p.max_logits[state]);
        }
        float local_sum = 0.0f;
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t part = begin + slice; part < end; part += SLICES) {
            const uint64_t state = ((uint64_t)part * p.num_q_heads + head) * max_q + local;
            const float part_sum = p.exp_sums[state];
            const float part_max = p.max_logits[state];
            // sliced-KV guards on isfinite(max), sliced-Q on sum == 0; both describe the empty partial.
            const bool empty = RANGED ? (part_sum == 0.0f) : !(fabsf(part_max) < INFINITY);
            const float weight = empty ? 0.0f : __expf(part_max - local_max) * part_sum;
            local_sum += weight;
            f32x4 value;
            if (p.partial_is_f32) {
                value = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.partial) + state * D + chunk * 4);
            } else {
                const uint2 bits = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.partial) + state * D + chunk * 4);
                value = f32x4{bf16_bits_to_f32(bits.x & 0xffffu), bf16_bits_to_f32(bits.x >> 16),
                              bf16_bits_to_f32(bits.y & 0xffffu), bf16_bits_to_f32(bits.y >> 16)};
            }
            if (weight != 0.0f) acc += value * weight;
        }
        if (chunk == 0) {
            slice_max[slice] = local_max;
            slice_sum[slice] = local_sum;
        }
        *reinterpret_cast<f32x4*>(&slice_acc[slice][chunk * 4]) = acc;
        __syncthreads();
        if (slice == 0) {
            float global_max = -INFINITY;
#pragma unroll
            for (int s = 0; s < SLICES; ++s) global_max = fmaxf(global_max, slice_max[s]);
            float global_sum = 0.0f;
            f32x4 total = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < SLICES; ++s) {
                if (slice_sum[s] > 0.0f) {
                    const float factor = __expf(slice_max[s] - global_max);
                    global_sum += slice_sum[s] * factor;
                    total += *reinterpret_cast<const f32x4*>(&slice_acc[s][chunk * 4]) * factor;
                }
            }
            f32x4 result = {0.0f, 0.0f, 0.0f, 0.0f};
            if (global_sum > 0.0f) result = total / global_sum;
            const uint64_t out_index = ((uint64_t)(flat_begin + local) * p.num_q_heads + head) * D + chunk * 4;
            if (p.gates != nullptr) {
                const uint2 gate_bits = *reinterpret_cast<const uint2*>(p.gates + out_index);
                const float gate[4] = {bf16_bits_to_f32(gate_bits.x & 0xffffu), bf16_bits_to_f32(gate_bits.x >> 16),
                                       bf16_bits_to_f32(gate_bits.y & 0xffffu), bf16_bits_to_f32(gate_bits.y >> 16)};
#pragma unroll
                for (int i = 0; i < 4; ++i) result[i] = round_to_bf16(result[i]) * sigmoid_bf16_steps(gate[i]);
            }
            const uint2 packed = make_uint2(pack_bf16x2(result[0], result[1]), pack_bf16x2(result[2], result[3]));
            *reinterpret_cast<uint2*>(p.output + out_index) = packed;
        }
        __syncthreads();
    }
}

// gqa_activation_gate_{f32,bf16} (gqa_activation_gate.metal:28-59): one thread per element.
__global__ __launch_bounds__(256) void activation_gate_kernel(const GateParams p) {
    const uint64_t total = (uint64_t)resolve_u32(p.num_active_tokens, p.replay_parameters) * p.values_per_token;
    const uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= total) return;
    if (p.is_f32) {
        const float a = reinterpret_cast<const float*>(p.attention)[gid];
        const float x = reinterpret_cast<const float*>(p.gates)[gid];
        reinterpret_cast<float*>(p.output)[gid] = a * sigmoid_f32(x);
    } else {
        const float a = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.attention)[gid]);
        const float x = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.gates)[gid]);
        reinterpret_cast<uint16_t*>(p.output)[gid] = f32_to_bf16_bits(a * sigmoid_bf16_steps(x));
    }
}

}  // namespace khm
