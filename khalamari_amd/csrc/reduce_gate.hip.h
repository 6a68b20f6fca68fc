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

#include "device_math.hip.h"
#include "device_params.h"
#include "lse_merge.hip.h"

namespace khm {

constexpr int kReduceThreads = 256;

// RANGED = false: sliced-KV flat reduce, grid (tokens, heads).
// RANGED = true : sliced-Q reduce, grid (Q ranges * max_q_tokens, heads): one block per token slot of a range, so the
//                 tokens of a range reduce side by side rather than in a serial loop of dependent loads.
template <int D, bool RANGED>
__global__ __launch_bounds__(kReduceThreads) void split_kv_reduce_kernel(const ReduceParams p) {
    constexpr int CHUNKS = D / 4;                    // threads per row
    constexpr int SLICES = kReduceThreads / CHUNKS;  // partial slices per block
    __shared__ float slice_stats[SLICES * 2];
    __shared__ __align__(16) float slice_acc[SLICES * D];

    const uint32_t unit = RANGED ? blockIdx.x / p.max_q_tokens : blockIdx.x;
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
    const uint32_t slice = threadIdx.x / CHUNKS;

    const uint32_t local = RANGED ? blockIdx.x - unit * p.max_q_tokens : 0u;
    if (local >= num_q) return;
    {
        MergeState state = merge_state_empty();
        if (end > begin) {
            merge_partial_slice<D, false>(state, p.max_logits, p.exp_sums, p.partial, p.partial_is_f32 != 0, begin + slice, end, SLICES, begin,
                                          p.num_q_heads, head, max_q, local, chunk);
        }
        if (chunk == 0) {
            slice_stats[slice * 2] = state.run_max;
            slice_stats[slice * 2 + 1] = state.run_sum;
        }
        *reinterpret_cast<f32x4*>(slice_acc + slice * D + chunk * 4) = state.acc;
        __syncthreads();
        if (slice == 0) {
            const MergeState total = merge_combine_slices<D>(slice_stats, slice_acc, 0, SLICES, chunk);
            const uint64_t out_index = ((uint64_t)(flat_begin + local) * p.num_q_heads + head) * D + chunk * 4;
            merge_store_output(total, p.output, p.gates, out_index);
        }
    }
}

// The same merge for rows with few partials (speculative-verify tiles have about ten): a group of D/4 threads owns one
// (token, head) row and walks all of its partials itself, sixteen loads in flight (a row of a decode batch with 512-token
// partitions has up to sixteen partials), so a block serves 256 / (D/4) rows and nothing passes through LDS.  Rows are numbered (unit * max_q_tokens + token slot) * num_q_heads + head.
template <int D, bool RANGED>
__global__ __launch_bounds__(kReduceThreads) void split_kv_reduce_rows_kernel(const ReduceParams p) {
    constexpr int CHUNKS = D / 4;
    constexpr int ROWS = kReduceThreads / CHUNKS;
    const int chunk = threadIdx.x % CHUNKS;
    const uint64_t row = (uint64_t)blockIdx.x * ROWS + threadIdx.x / CHUNKS;
    const uint32_t max_q = RANGED ? p.max_q_tokens : 1u;
    const uint64_t slot = row / p.num_q_heads;
    const uint32_t head = (uint32_t)(row - slot * p.num_q_heads);
    const uint32_t unit = (uint32_t)(slot / max_q);
    const uint32_t local = (uint32_t)(slot - (uint64_t)unit * max_q);
    if (unit >= resolve_u32(p.num_active, p.replay_parameters)) return;
    uint32_t flat_begin = unit, num_q = 1;
    if (RANGED) {
        flat_begin = p.q_token_ranges[2 * (uint64_t)unit];
        num_q = p.q_token_ranges[2 * (uint64_t)unit + 1] - flat_begin;
        if (num_q > max_q) num_q = max_q;
    }
    if (local >= num_q) return;
    const uint32_t begin = p.cu_partial_outputs[unit];
    const uint32_t end = p.cu_partial_outputs[unit + 1];
    MergeState state = merge_state_empty();
    if (end > begin) {
        merge_partial_slice<D, false, 16>(state, p.max_logits, p.exp_sums, p.partial, p.partial_is_f32 != 0, begin, end, 1, begin, p.num_q_heads, head,
                                      max_q, local, chunk);
    }
    const uint64_t out_index = ((uint64_t)(flat_begin + local) * p.num_q_heads + head) * D + chunk * 4;
    merge_store_output(state, p.output, p.gates, out_index);
}

// gqa_activation_gate_{f32,bf16} (gqa_activation_gate.metal:28-59): one thread per element.  For buffers that are not
// 16-byte aligned; the vector kernel below is the one that normally runs.
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

// The same arithmetic, 16 bytes per thread and buffer (eight bf16 or four f32 elements), the output written with streaming
// stores (it is read by the next launch, not by this one); what is left of the last group goes element by element.
constexpr int gate_elements_per_thread(bool f32) { return f32 ? 4 : 8; }
template <bool F32>
__global__ __launch_bounds__(256) void activation_gate_vector_kernel(const GateParams p) {
    constexpr int EPT = gate_elements_per_thread(F32);
    const uint64_t total = (uint64_t)resolve_u32(p.num_active_tokens, p.replay_parameters) * p.values_per_token;
    const uint64_t first = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * EPT;
    if (first >= total) return;
    if (first + EPT <= total) {
        if constexpr (F32) {
            const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.attention) + first);
            const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.gates) + first);
            store_streaming(reinterpret_cast<float*>(p.output) + first,
                            make_float4(a.x * sigmoid_f32(x.x), a.y * sigmoid_f32(x.y), a.z * sigmoid_f32(x.z), a.w * sigmoid_f32(x.w)));
        } else {
            const uint4 a = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.attention) + first);
            const uint4 x = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.gates) + first);
            const uint32_t a_words[4] = {a.x, a.y, a.z, a.w}, x_words[4] = {x.x, x.y, x.z, x.w};
            uint32_t out[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float low = bf16_bits_to_f32(a_words[i] & 0xffffu) * sigmoid_bf16_steps(bf16_bits_to_f32(x_words[i] & 0xffffu));
                const float high = bf16_bits_to_f32(a_words[i] >> 16) * sigmoid_bf16_steps(bf16_bits_to_f32(x_words[i] >> 16));
                out[i] = pack_bf16x2(low, high);
            }
            store_streaming(reinterpret_cast<uint16_t*>(p.output) + first, make_uint4(out[0], out[1], out[2], out[3]));
        }
        return;
    }
    for (uint64_t i = first; i < total; ++i) {
        if constexpr (F32) {
            reinterpret_cast<float*>(p.output)[i] = reinterpret_cast<const float*>(p.attention)[i] * sigmoid_f32(reinterpret_cast<const float*>(p.gates)[i]);
        } else {
            const float a = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.attention)[i]);
            const float x = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.gates)[i]);
            reinterpret_cast<uint16_t*>(p.output)[i] = f32_to_bf16_bits(a * sigmoid_bf16_steps(x));
        }
    }
}

}  // namespace khm
