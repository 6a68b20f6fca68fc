// Dense bidirectional block SDPA that writes one partial state into the split-KV partial-output layout.
//
// Mirrors bidi_block_sdpa::{Config, Shape, Buffers, Compute, Invocation}
// (crates/inference-backend-metal/src/components/gqa/bidi_block_sdpa.rs:44-340) and the kernels
// gqa_bidi_block_sdpa_{f32,bf16} (.../metal/gqa_bidi_block_sdpa.metal:10-126): every Q token attends, without a mask,
// to the `block_size` local K/V tokens of its own request block; the result lands in the last partial slot of the
// token's Q range (cu_sdpa_partial_outputs[range + 1] - 1), where the sliced-Q Reduce merges it with the history
// partials.  Stored maxima are natural-log, like every partial of this ABI.
//
// Work shape on gfx950.  One 256-thread block per (Q range, KV head): the K and V rows of the request block under that KV
// head are staged once in LDS as f32 (16-byte global loads, every Q head of the group and every token of the range reads
// them from there), and the block's (token, Q head) tasks are served sixteen at a time, one task per 16-lane row of a
// wave.  A lane keeps its eight-dim chunks of the Q row in registers (one 16-byte load per 128 dims), scores are dot
// products over the lane's chunks summed across the row with DPP rotations, and the weighted V sum accumulates in
// registers, eight dims per lane and chunk, stored with 16-byte stores.  Keys are walked in LDS-sized tiles with a
// running maximum; a request block that fits one tile (the case the executor produces) is the reference's two passes:
// maximum first, then weights, their sum and the weighted sum in key order.
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

// Sum over the sixteen lanes of a row, result in every lane of the row (DPP row rotations, no LDS).
__device__ __forceinline__ float sum_within_row(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, true));   // row_ror:8
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x124, 0xf, 0xf, true));   // row_ror:4
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x122, 0xf, 0xf, true));   // row_ror:2
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x121, 0xf, 0xf, true));   // row_ror:1
    return x;
}

// Eight consecutive values of a row as f32; T = float or uint16_t (bf16 bits).  `base` + `index` is 16-byte aligned.
template <typename T>
__device__ __forceinline__ void load_chunk(const void* base, uint64_t index, float (&out)[8]);
template <>
__device__ __forceinline__ void load_chunk<float>(const void* base, uint64_t index, float (&out)[8]) {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + index);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + index + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[i] = lo[i];
        out[4 + i] = hi[i];
    }
}
template <>
__device__ __forceinline__ void load_chunk<uint16_t>(const void* base, uint64_t index, float (&out)[8]) {
    const uint4 bits = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + index);
    const uint32_t words[4] = {bits.x, bits.y, bits.z, bits.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = bf16_bits_to_f32(words[i] & 0xffffu);
        out[2 * i + 1] = bf16_bits_to_f32(words[i] >> 16);
    }
}
__device__ __forceinline__ void store_chunk(float* base, uint64_t index, const float (&value)[8]) {
    *reinterpret_cast<f32x4*>(base + index) = f32x4{value[0], value[1], value[2], value[3]};
    *reinterpret_cast<f32x4*>(base + index + 4) = f32x4{value[4], value[5], value[6], value[7]};
}
__device__ __forceinline__ void store_chunk(uint16_t* base, uint64_t index, const float (&value)[8]) {
    *reinterpret_cast<uint4*>(base + index) = make_uint4(pack_bf16x2(value[0], value[1]), pack_bf16x2(value[2], value[3]),
                                                         pack_bf16x2(value[4], value[5]), pack_bf16x2(value[6], value[7]));
}

constexpr int kBidiThreads = 256;
constexpr int kBidiTasksPerRound = kBidiThreads / 16;

// T = float or uint16_t (bf16 bits); CHUNKS = ceil(head_dim / 128): eight-dim chunks per lane.  Dynamic LDS: K and V of
// one key tile as f32, 2 * key_tile * head_dim floats.
template <typename T, int CHUNKS>
__global__ __launch_bounds__(kBidiThreads) void bidi_block_sdpa_kernel(const BidiBlockParams p, uint32_t key_tile) {
    extern __shared__ __align__(16) float staged[];
    const uint32_t range = blockIdx.x;
    const uint32_t kv_head = blockIdx.y;
    if (range >= resolve_u32(p.num_active_q_token_ranges, p.replay_parameters)) return;
    const uint32_t flat_begin = p.q_token_ranges[2 * (uint64_t)range];
    const uint32_t flat_end = p.q_token_ranges[2 * (uint64_t)range + 1];
    // ranges and cumulative counts come from device memory: anything that points outside the buffers is skipped
    if (flat_end <= flat_begin || flat_end > p.num_total_tokens) return;
    uint32_t num_q = flat_end - flat_begin;
    if (num_q > p.max_q_tokens) num_q = p.max_q_tokens;
    const uint32_t slot = p.cu_partial_outputs[range + 1] - 1;
    if (slot >= p.num_total_partial_output_slots) return;

    const uint32_t D = p.head_dim, B = p.block_size;
    const uint32_t group = p.num_q_heads / p.num_kv_heads;
    const uint32_t tid = threadIdx.x;
    const uint32_t sub = tid & 15;                      // lane within the task's row
    const uint32_t row_in_block = tid >> 4;             // which of the sixteen tasks of a round
    float* k_lds = staged;                              // [key_tile][D]
    float* v_lds = staged + (uint64_t)key_tile * D;
    bool chunk_live[CHUNKS];
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) chunk_live[j] = (j * 16 + sub) * 8 < D;

    // the tokens of a range lie in one request block when the executor built the ranges; any range is handled
    const uint32_t first_block = flat_begin / B, last_block = (flat_begin + num_q - 1) / B;
    for (uint32_t request_block = first_block; request_block <= last_block; ++request_block) {
        const uint32_t local_begin = request_block * B;
        const uint32_t token_lo = local_begin > flat_begin ? local_begin : flat_begin;
        const uint32_t token_hi = local_begin + B < flat_begin + num_q ? local_begin + B : flat_begin + num_q;
        const uint32_t num_tasks = (token_hi - token_lo) * group;
        auto stage_tile = [&](uint32_t tile_begin, uint32_t tile_keys) __attribute__((always_inline)) {
            __syncthreads();   // everyone is done with what the tile buffers held
            for (uint32_t index = tid; index < tile_keys * (D / 8); index += kBidiThreads) {
                const uint32_t key = index / (D / 8), chunk = index % (D / 8);
                const uint64_t source = ((uint64_t)(local_begin + tile_begin + key) * p.num_kv_heads + kv_head) * D + chunk * 8;
                float values[8];
                load_chunk<T>(p.local_k, source, values);
                store_chunk(k_lds, (uint64_t)key * D + chunk * 8, values);
                load_chunk<T>(p.local_v, source, values);
                store_chunk(v_lds, (uint64_t)key * D + chunk * 8, values);
            }
            __syncthreads();
        };
        // a request block that fits the tile buffers is staged once for all rounds of tasks
        const bool single_tile = key_tile >= B;
        if (single_tile) stage_tile(0, B);
        for (uint32_t round = 0; round * kBidiTasksPerRound < num_tasks; ++round) {
            const uint32_t task = round * kBidiTasksPerRound + row_in_block;
            const bool live = task < num_tasks;
            const uint32_t q_token = token_lo + (live ? task / group : 0u);
            const uint32_t q_head = kv_head * group + (live ? task % group : 0u);
            float q[CHUNKS][8], acc[CHUNKS][8];
            const uint64_t q_row = ((uint64_t)q_token * p.num_q_heads + q_head) * D;
#pragma unroll
            for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
                for (int i = 0; i < 8; ++i) q[j][i] = acc[j][i] = 0.0f;
                if (chunk_live[j]) load_chunk<T>(p.q, q_row + (j * 16 + sub) * 8, q[j]);
            }
            float run_max = -INFINITY, run_sum = 0.0f;
            for (uint32_t tile_begin = 0; tile_begin < B; tile_begin += key_tile) {
                const uint32_t tile_keys = B - tile_begin < key_tile ? B - tile_begin : key_tile;
                if (!single_tile) stage_tile(tile_begin, tile_keys);
                auto score_of = [&](uint32_t key) __attribute__((always_inline)) -> float {
                    float part = 0.0f;
#pragma unroll
                    for (int j = 0; j < CHUNKS; ++j) {
                        if (chunk_live[j]) {
                            float k_values[8];
                            load_chunk<float>(k_lds, (uint64_t)key * D + (j * 16 + sub) * 8, k_values);
#pragma unroll
                            for (int i = 0; i < 8; ++i) part = __builtin_fmaf(q[j][i], k_values[i], part);
                        }
                    }
                    return sum_within_row(part) * p.scale;
                };
                float tile_max = -INFINITY;
                for (uint32_t key = 0; key < tile_keys; ++key) tile_max = fmaxf(tile_max, score_of(key));
                const float next_max = fmaxf(run_max, tile_max);
                const float keep = __expf(run_max - next_max);   // 0 before the first tile
                run_sum *= keep;
#pragma unroll
                for (int j = 0; j < CHUNKS; ++j)
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[j][i] *= keep;
                run_max = next_max;
                for (uint32_t key = 0; key < tile_keys; ++key) {
                    const float weight = __expf(score_of(key) - run_max);
                    run_sum += weight;
#pragma unroll
                    for (int j = 0; j < CHUNKS; ++j) {
                        if (chunk_live[j]) {
                            float v_values[8];
                            load_chunk<float>(v_lds, (uint64_t)key * D + (j * 16 + sub) * 8, v_values);
#pragma unroll
                            for (int i = 0; i < 8; ++i) acc[j][i] = __builtin_fmaf(weight, v_values[i], acc[j][i]);
                        }
                    }
                }
            }
            if (live) {
                const uint64_t state = ((uint64_t)slot * p.num_q_heads + q_head) * p.max_q_tokens + (q_token - flat_begin);
                if (sub == 0) {
                    p.exp_sums[state] = run_sum;
                    p.max_logits[state] = run_max;
                }
                const float inverse = run_sum > 0.0f ? 1.0f / run_sum : 0.0f;
#pragma unroll
                for (int j = 0; j < CHUNKS; ++j) {
                    if (chunk_live[j]) {
                        float values[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) values[i] = acc[j][i] * inverse;
                        store_chunk(static_cast<T*>(p.partial_output), state * D + (j * 16 + sub) * 8, values);
                    }
                }
            }
        }
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
    KHM_REQUIRE(config->num_kv_heads <= 65535, "bidirectional block SDPA grid exceeds 65535 KV heads");
    if (config->head_dim > 1024) return fail(KHM_ERR_UNSUPPORTED, "no gfx950 bidirectional block SDPA kernel for head_dim %u (at most 1024)", config->head_dim);
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
    // key tile: as many keys as 48 KB of LDS hold as f32 K and V rows (a whole request block in every executor shape)
    const uint32_t lds_budget = 48 * 1024;
    uint32_t key_tile = lds_budget / (2 * config->head_dim * 4);
    if (key_tile > config->block_size) key_tile = config->block_size;
    const uint32_t lds_bytes = 2 * key_tile * config->head_dim * 4;
    const dim3 grid(shape->num_total_q_token_ranges, config->num_kv_heads, 1);
    const uint32_t chunks = (config->head_dim + 127) / 128;
    typedef void (*Kernel)(const BidiBlockParams, uint32_t);
    Kernel kernel = nullptr;
    const bool f32 = config->dtype == KHM_DTYPE_F32;
    if (chunks <= 1) kernel = f32 ? bidi_block_sdpa_kernel<float, 1> : bidi_block_sdpa_kernel<uint16_t, 1>;
    else if (chunks <= 2) kernel = f32 ? bidi_block_sdpa_kernel<float, 2> : bidi_block_sdpa_kernel<uint16_t, 2>;
    else if (chunks <= 4) kernel = f32 ? bidi_block_sdpa_kernel<float, 4> : bidi_block_sdpa_kernel<uint16_t, 4>;
    else kernel = f32 ? bidi_block_sdpa_kernel<float, 8> : bidi_block_sdpa_kernel<uint16_t, 8>;
    KHM_LAUNCH(kernel, grid, dim3(kBidiThreads), lds_bytes, static_cast<hipStream_t>(stream), p, key_tile);
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "bidirectional block SDPA launch failed: %s", hipGetErrorString(status));
    return KHM_OK;
}
