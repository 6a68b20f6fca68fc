// Dense bidirectional block SDPA that writes one partial state into the split-KV partial-output layout.
//
// Mirrors bidi_block_sdpa::{Config, Shape, Buffers, Compute, Invocation}
// (crates/inference-backend-metal/src/components/gqa/bidi_block_sdpa.rs:44-340) and the kernels
// gqa_bidi_block_sdpa_{f32,bf16} (.../metal/gqa_bidi_block_sdpa.metal:10-126): every Q token attends, without a mask,
// to the `block_size` local K/V tokens of its own request block; the result lands in the last partial slot of the
// token's Q range (cu_sdpa_partial_outputs[range + 1] - 1), where the sliced-Q Reduce merges it with the history
// partials.  Stored maxima are natural-log, like every partial of this ABI.
//
// One wavefront per (Q head, Q range, token offset), as in the reference (one SIMDgroup there): the work per task is
// block_size x head_dim, far too little to tile; lanes stride over the head dimension.
#include <hip/hip_runtime.h>

#include "common.h"
#include "device_math.hip.h"
#include "device_params.h"

namespace khm {

struct BidiBlockParams {
    const void* q;                          // [T][Hq][D]
    const void* local_k;                    // [T][Hkv][D]
    const void* local_v;
    const uint32_t* q_token_ranges;         // [R][2]
    const uint32_t* cu_partial_outputs;     // [R + 1]
    float* exp_sums;                        // [slots][Hq][max_q_tokens]
    float* max_logits;
    void* partial_output;                   // [slots][Hq][max_q_tokens][D]
    const uint32_t* replay_parameters;
    DeviceReplayU32 num_active_q_token_ranges;
    uint32_t num_total_tokens;
    uint32_t num_total_partial_output_slots;
    uint32_t block_size;
    uint32_t max_q_tokens;
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    float scale;
};

template <typename T>
__device__ __forceinline__ float load_value(const void* base, uint64_t index);
template <>
__device__ __forceinline__ float load_value<float>(const void* base, uint64_t index) {
    return static_cast<const float*>(base)[index];
}
template <>
__device__ __forceinline__ float load_value<uint16_t>(const void* base, uint64_t index) {
    return bf16_bits_to_f32(static_cast<const uint16_t*>(base)[index]);
}
__device__ __forceinline__ void store_value(float* base, uint64_t index, float value) { base[index] = value; }
__device__ __forceinline__ void store_value(uint16_t* base, uint64_t index, float value) { base[index] = f32_to_bf16_bits(value); }

// T = float or uint16_t (bf16 bits).  Dynamic LDS: block_size floats (the logits, then the weights).
template <typename T>
__global__ __launch_bounds__(64) void bidi_block_sdpa_kernel(const BidiBlockParams p) {
    extern __shared__ float block_logits[];
    const uint32_t lane = threadIdx.x;
    const uint32_t q_head = blockIdx.x;
    const uint32_t range = blockIdx.y;
    if (range >= resolve_u32(p.num_active_q_token_ranges, p.replay_parameters)) return;
    const uint32_t offset = blockIdx.z;
    const uint32_t flat_begin = p.q_token_ranges[2 * (uint64_t)range];
    const uint32_t flat_end = p.q_token_ranges[2 * (uint64_t)range + 1];
    // ranges and cumulative counts come from device memory: anything that points outside the buffers is skipped
    if (flat_end <= flat_begin || flat_end > p.num_total_tokens || offset >= flat_end - flat_begin) return;
    const uint32_t q_token = flat_begin + offset;
    const uint32_t kv_head = q_head / (p.num_q_heads / p.num_kv_heads);
    const uint32_t local_begin = (q_token / p.block_size) * p.block_size;
    const uint32_t slot = p.cu_partial_outputs[range + 1] - 1;
    if (slot >= p.num_total_partial_output_slots) return;
    const uint64_t q_row = ((uint64_t)q_token * p.num_q_heads + q_head) * p.head_dim;

    for (uint32_t local = 0; local < p.block_size; ++local) {
        const uint64_t k_row = ((uint64_t)(local_begin + local) * p.num_kv_heads + kv_head) * p.head_dim;
        float score = 0.0f;
        for (uint32_t d = lane; d < p.head_dim; d += 64) score += load_value<T>(p.q, q_row + d) * load_value<T>(p.local_k, k_row + d);
#pragma unroll
        for (int step = 32; step >= 1; step >>= 1) score += __shfl_xor(score, step);
        if (lane == 0) block_logits[local] = score * p.scale;
    }
    __syncthreads();
    float block_max = -INFINITY;
    for (uint32_t local = 0; local < p.block_size; ++local) block_max = fmaxf(block_max, block_logits[local]);
    __syncthreads();
    // every lane derives the same weights; lane l rewrites entries l, l + 64, ...
    float exp_sum = 0.0f;
    for (uint32_t local = 0; local < p.block_size; ++local) exp_sum += __expf(block_logits[local] - block_max);
    for (uint32_t local = lane; local < p.block_size; local += 64) block_logits[local] = __expf(block_logits[local] - block_max);
    __syncthreads();
    const uint64_t state = ((uint64_t)slot * p.num_q_heads + q_head) * p.max_q_tokens + offset;
    if (lane == 0) {
        p.exp_sums[state] = exp_sum;
        p.max_logits[state] = block_max;
    }
    for (uint32_t d = lane; d < p.head_dim; d += 64) {
        float output = 0.0f;
        for (uint32_t local = 0; local < p.block_size; ++local) {
            const uint64_t v_index = ((uint64_t)(local_begin + local) * p.num_kv_heads + kv_head) * p.head_dim + d;
            output += block_logits[local] * load_value<T>(p.local_v, v_index);
        }
        store_value(static_cast<T*>(p.partial_output), state * p.head_dim + d, exp_sum > 0.0f ? output / exp_sum : 0.0f);
    }
}

}  // namespace khm

using namespace khm;

static bool product_fits_u32(uint64_t a, uint64_t b, uint64_t c = 1, uint64_t d = 1) {
    const __uint128_t product = (__uint128_t)a * b * c * d;
    return product <= 0xffffffffull;
}

extern "C" int khm_bidi_block_sdpa(const khm_bidi_block_sdpa_config* config, const khm_bidi_block_sdpa_shape* shape,
                                   const khm_bidi_block_sdpa_buffers* buffers, khm_replay_u32 num_active_q_token_ranges,
                                   const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(config != nullptr && shape != nullptr && buffers != nullptr, "config, shape and buffers must not be null");
    // Config::validate (bidi_block_sdpa.rs:66-82)
    KHM_REQUIRE(config->block_size > 0 && config->max_q_tokens > 0 && config->num_q_heads > 0 && config->num_kv_heads > 0 &&
                    config->head_dim > 0,
                "bidirectional block SDPA requires a block size, Q tokens, heads and a head dimension");
    KHM_REQUIRE(config->num_q_heads % config->num_kv_heads == 0, "bidirectional block SDPA Q heads must be a multiple of KV heads");
    KHM_REQUIRE(config->scale > 0.0f && config->scale < __builtin_inff(), "bidirectional block SDPA scale must be finite and positive");
    KHM_REQUIRE(config->head_dim % 32 == 0, "bidirectional block SDPA head_dim must be divisible by the SIMD width");
    KHM_REQUIRE(config->dtype == KHM_DTYPE_F32 || config->dtype == KHM_DTYPE_BF16, "unsupported bidirectional block SDPA dtype");
    // Shape::validate (bidi_block_sdpa.rs:148-173)
    KHM_REQUIRE(shape->num_total_tokens > 0, "bidirectional block SDPA requires tokens");
    KHM_REQUIRE(shape->num_total_q_token_ranges > 0 && shape->num_total_q_token_ranges <= shape->num_total_tokens,
                "bidirectional block SDPA Q-token ranges must be in 1..=num_total_tokens");
    KHM_REQUIRE(shape->num_total_partial_output_slots >= shape->num_total_q_token_ranges,
                "bidirectional block SDPA needs at least one partial-output slot per Q-token range");
    KHM_REQUIRE(shape->num_total_tokens % config->block_size == 0, "bidirectional block SDPA tokens must contain complete request blocks");
    KHM_REQUIRE(product_fits_u32(shape->num_total_tokens, config->num_q_heads, config->head_dim),
                "bidirectional block SDPA Q exceeds the shader u32 count domain");
    KHM_REQUIRE(product_fits_u32(shape->num_total_partial_output_slots, config->num_q_heads, config->max_q_tokens, config->head_dim),
                "bidirectional block SDPA partial output exceeds the shader u32 element-index domain");
    KHM_REQUIRE(config->max_q_tokens <= 65535 && shape->num_total_q_token_ranges <= 65535,
                "bidirectional block SDPA grid exceeds 65535 in y or z");
    KHM_REQUIRE((uint64_t)config->block_size * 4 <= 64 * 1024, "bidirectional block SDPA requires %u bytes of thread-block memory",
                config->block_size * 4);
    // Invocation::validate (bidi_block_sdpa.rs:289-333)
    if (!num_active_q_token_ranges.is_parameter) {
        KHM_REQUIRE(num_active_q_token_ranges.value == shape->num_total_q_token_ranges,
                    "a fixed num_active_q_token_ranges must equal num_total_q_token_ranges");
    } else {
        KHM_REQUIRE(replay_parameters != nullptr, "num_active_q_token_ranges is a replay parameter but no parameter block was given");
    }
    const uint64_t item = dtype_item_size(config->dtype);
    const uint64_t q_bytes = (uint64_t)shape->num_total_tokens * config->num_q_heads * config->head_dim * item;
    const uint64_t kv_bytes = (uint64_t)shape->num_total_tokens * config->num_kv_heads * config->head_dim * item;
    const uint64_t stats = (uint64_t)shape->num_total_partial_output_slots * config->num_q_heads * config->max_q_tokens;
#define KHM_BIDI_AT_LEAST(buffer, bytes, name)                                                                                  \
    KHM_REQUIRE((buffer).ptr != nullptr && (buffer).len_bytes >= (uint64_t)(bytes), "%s buffer holds %llu bytes, needs %llu", name, \
                (unsigned long long)(buffer).len_bytes, (unsigned long long)(bytes))
    KHM_BIDI_AT_LEAST(buffers->q, q_bytes, "q");
    KHM_BIDI_AT_LEAST(buffers->local_k, kv_bytes, "local_k");
    KHM_BIDI_AT_LEAST(buffers->local_v, kv_bytes, "local_v");
    KHM_BIDI_AT_LEAST(buffers->q_token_ranges, (uint64_t)shape->num_total_q_token_ranges * 8, "q_token_ranges");
    KHM_BIDI_AT_LEAST(buffers->cu_sdpa_partial_outputs, ((uint64_t)shape->num_total_q_token_ranges + 1) * 4, "cu_sdpa_partial_outputs");
    KHM_BIDI_AT_LEAST(buffers->partial_exp_sums, stats * 4, "partial_exp_sums");
    KHM_BIDI_AT_LEAST(buffers->partial_max_logits, stats * 4, "partial_max_logits");
    KHM_BIDI_AT_LEAST(buffers->partial_output, stats * config->head_dim * item, "partial_output");
#undef KHM_BIDI_AT_LEAST

    BidiBlockParams p{};
    p.q = buffers->q.ptr;
    p.local_k = buffers->local_k.ptr;
    p.local_v = buffers->local_v.ptr;
    p.q_token_ranges = static_cast<const uint32_t*>(buffers->q_token_ranges.ptr);
    p.cu_partial_outputs = static_cast<const uint32_t*>(buffers->cu_sdpa_partial_outputs.ptr);
    p.exp_sums = static_cast<float*>(buffers->partial_exp_sums.ptr);
    p.max_logits = static_cast<float*>(buffers->partial_max_logits.ptr);
    p.partial_output = buffers->partial_output.ptr;
    p.replay_parameters = replay_parameters;
    p.num_active_q_token_ranges = DeviceReplayU32{num_active_q_token_ranges.is_parameter, num_active_q_token_ranges.value};
    p.num_total_tokens = shape->num_total_tokens;
    p.num_total_partial_output_slots = shape->num_total_partial_output_slots;
    p.block_size = config->block_size;
    p.max_q_tokens = config->max_q_tokens;
    p.num_q_heads = config->num_q_heads;
    p.num_kv_heads = config->num_kv_heads;
    p.head_dim = config->head_dim;
    p.scale = config->scale;
    const dim3 grid(config->num_q_heads, shape->num_total_q_token_ranges, config->max_q_tokens);
    const uint32_t lds_bytes = config->block_size * 4;
    if (config->dtype == KHM_DTYPE_F32) {
        hipLaunchKernelGGL(bidi_block_sdpa_kernel<float>, grid, dim3(64), lds_bytes, static_cast<hipStream_t>(stream), p);
    } else {
        hipLaunchKernelGGL(bidi_block_sdpa_kernel<uint16_t>, grid, dim3(64), lds_bytes, static_cast<hipStream_t>(stream), p);
    }
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "bidirectional block SDPA launch failed: %s", hipGetErrorString(status));
    return KHM_OK;
}
