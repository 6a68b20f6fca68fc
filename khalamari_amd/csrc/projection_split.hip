// Split of the fused input projection into the Q, (gate,) K and V rows the rest of the layer reads.
//
// Mirrors qgkv_split::{Config, Shape, Buffers, Compute, Invocation}
// (crates/inference-backend-metal/src/components/gqa/qgkv_split.rs:34-236, kernel .../metal/gqa_qgkv_split.metal:5-44) and
// qkv_split::{...} (.../gqa/qkv_split.rs, kernel .../metal/gqa_qkv_split.metal:5-34): a token's projection row is
// [Hq x (q head | gate head)][Hkv x k head][Hkv x v head] in the gated form and [Hq x q head][Hkv x k][Hkv x v] in the
// ungated one; the first num_active_tokens rows are scattered to q [T][Hq][D], g [T][Hq][D], k and v [T][Hkv][D].
// Pure data movement, bit-exact.  Nothing here allocates or synchronizes.
#include <hip/hip_runtime.h>

#include "common.h"
#include "device_math.hip.h"
#include "device_params.h"

namespace khm {

struct SplitParams {
    const void* projection;             // [T][row_units] units
    void* q;                            // [T][Hq * head_units]
    void* g;                            // [T][Hq * head_units], gated form only
    void* k;                            // [T][Hkv * head_units]
    void* v;                            // [T][Hkv * head_units]
    const uint32_t* replay_parameters;
    DeviceReplayU32 num_active_tokens;
    uint32_t head_units;                // units per head row
    uint32_t q_units;                   // Hq * head_units
    uint32_t kv_units;                  // Hkv * head_units
    uint32_t row_units;                 // (1 or 2) * q_units + 2 * kv_units
    uint32_t row_blocks;                // blocks of 256 units per row
};

// Every boundary inside a projection row is a multiple of one head row, so the copy works in units of up to 16 bytes that
// divide a head row.  A block moves 256 consecutive units of one token's row, and consecutive blocks continue along the
// row and then into the next token: the launch sweeps the projection front to back, and each of the four outputs front to
// back.  Every byte is touched once: streaming loads and stores.  Measured on 16384 tokens of Hq 64 / Hkv 8 / D 128 bf16
// (604 MB in, 604 MB out): 193 us = 78 % of 8 TB/s; 220 us with ordinary loads and stores; 260 us with the same blocks
// ordered token-fastest, four tokens per block (neighbouring blocks 144 KB apart); two to nine units or two to eight tokens per thread: 195-209 us.
template <typename Unit>
__device__ __forceinline__ Unit load_unit_streaming(const Unit* source) {
    return __builtin_nontemporal_load(source);
}
template <>
__device__ __forceinline__ uint4 load_unit_streaming<uint4>(const uint4* source) {
    return load_streaming(source);
}
template <>
__device__ __forceinline__ uint2 load_unit_streaming<uint2>(const uint2* source) {
    typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));
    const U32x2 value = __builtin_nontemporal_load(reinterpret_cast<const U32x2*>(source));
    return make_uint2(value.x, value.y);
}
template <typename Unit>
__device__ __forceinline__ void store_unit_streaming(Unit* target, Unit value) {
    __builtin_nontemporal_store(value, target);
}
template <>
__device__ __forceinline__ void store_unit_streaming<uint4>(uint4* target, uint4 value) {
    store_streaming(target, value);
}
template <>
__device__ __forceinline__ void store_unit_streaming<uint2>(uint2* target, uint2 value) {
    store_streaming(target, value);
}

// Where unit position `unit` of a projection row goes: gqa_qgkv_split.metal:24-43 / gqa_qkv_split.metal:22-33 in units of a
// head row's divisor.
template <typename Unit>
struct SplitTarget {
    Unit* base;          // the destination buffer, advanced to the unit's place in token 0's row
    uint32_t row_units;  // units per token row of that buffer
};

template <typename Unit, bool GATED>
__device__ __forceinline__ SplitTarget<Unit> split_target_of(const SplitParams& p, uint32_t unit) {
    const uint32_t query_units = GATED ? 2 * p.q_units : p.q_units;
    if (unit < query_units) {
        if (GATED) {
            const uint32_t pair = unit / (2 * p.head_units);
            const uint32_t in_pair = unit - pair * 2 * p.head_units;
            const bool gate = in_pair >= p.head_units;
            return {static_cast<Unit*>(gate ? p.g : p.q) + pair * p.head_units + (gate ? in_pair - p.head_units : in_pair), p.q_units};
        }
        return {static_cast<Unit*>(p.q) + unit, p.q_units};
    }
    if (unit < query_units + p.kv_units) return {static_cast<Unit*>(p.k) + (unit - query_units), p.kv_units};
    return {static_cast<Unit*>(p.v) + (unit - query_units - p.kv_units), p.kv_units};
}

template <typename Unit, bool GATED>
__global__ __launch_bounds__(256) void projection_split_kernel(const SplitParams p) {
    const uint32_t num_active = resolve_u32(p.num_active_tokens, p.replay_parameters);
    const uint32_t token = blockIdx.x / p.row_blocks;
    if (token >= num_active) return;
    const uint32_t unit = (blockIdx.x - token * p.row_blocks) * 256 + threadIdx.x;
    if (unit >= p.row_units) return;
    const Unit value = load_unit_streaming(static_cast<const Unit*>(p.projection) + (uint64_t)token * p.row_units + unit);
    const SplitTarget<Unit> target = split_target_of<Unit, GATED>(p, unit);
    store_unit_streaming(target.base + (uint64_t)token * target.row_units, value);
}

static uint64_t item_size(uint32_t dtype) { return dtype == KHM_DTYPE_F32 ? 4 : 2; }

// Largest power of two up to 16 bytes that divides a head row and every buffer address.
static uint32_t unit_bytes_for(uint64_t head_row_bytes, const khm_buffer* const* buffers, int count) {
    uint64_t bits = head_row_bytes | 16;
    for (int i = 0; i < count; ++i) bits |= reinterpret_cast<uintptr_t>(buffers[i]->ptr);
    return (uint32_t)(bits & (~bits + 1));
}

template <bool GATED>
static void launch_split(uint32_t unit_bytes, dim3 grid, hipStream_t stream, const SplitParams& p) {
    switch (unit_bytes) {
        case 16: KHM_LAUNCH((projection_split_kernel<uint4, GATED>), grid, dim3(256), 0, stream, p); break;
        case 8: KHM_LAUNCH((projection_split_kernel<uint2, GATED>), grid, dim3(256), 0, stream, p); break;
        case 4: KHM_LAUNCH((projection_split_kernel<uint32_t, GATED>), grid, dim3(256), 0, stream, p); break;
        default: KHM_LAUNCH((projection_split_kernel<uint16_t, GATED>), grid, dim3(256), 0, stream, p); break;
    }
}

static int projection_split(bool gated, const khm_gqa_projection_split_config* config, uint32_t num_total_tokens,
                            const khm_buffer& projection, const khm_buffer& q, const khm_buffer* g, const khm_buffer& k,
                            const khm_buffer& v, khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    const char* what = gated ? "GQA projection" : "ungated GQA projection";
    KHM_REQUIRE(config != nullptr, "config must not be null");
    // Config::validate (qgkv_split.rs:61-67, qkv_split.rs)
    KHM_REQUIRE(config->num_q_heads > 0 && config->num_kv_heads > 0 && config->head_dim > 0,
                "%s split requires Q heads, KV heads and a head dimension", what);
    KHM_REQUIRE(config->dtype == KHM_DTYPE_F32 || config->dtype == KHM_DTYPE_BF16, "unsupported GQA projection split dtype %u", config->dtype);
    const uint64_t row_heads = (gated ? 2ull : 1ull) * config->num_q_heads + 2ull * config->num_kv_heads;
    KHM_REQUIRE(row_heads <= 0xffffffffull, "GQA fused projection head count must fit u32");
    // Shape::validate (qgkv_split.rs:141-146): the reference indexes elements with one u32
    KHM_REQUIRE(num_total_tokens > 0, "%s split requires tokens", what);
    const __uint128_t elements = (__uint128_t)num_total_tokens * row_heads * config->head_dim;
    KHM_REQUIRE(elements <= 0xffffffffull, "%s elements exceeds the shader u32 count domain", what);
    // Invocation::validate (qgkv_split.rs:224-235)
    if (!num_active_tokens.is_parameter) {
        KHM_REQUIRE(num_active_tokens.value >= 1 && num_active_tokens.value <= num_total_tokens,
                    "num_active_tokens=%u is outside its replay domain [1, %u]", num_active_tokens.value, num_total_tokens);
    } else {
        KHM_REQUIRE(replay_parameters != nullptr, "num_active_tokens is a replay parameter but no parameter block was given");
    }
    const uint64_t item = item_size(config->dtype);
    const uint64_t head_row_bytes = (uint64_t)config->head_dim * item;
    const uint64_t q_bytes = (uint64_t)num_total_tokens * config->num_q_heads * head_row_bytes;
    const uint64_t kv_bytes = (uint64_t)num_total_tokens * config->num_kv_heads * head_row_bytes;
    const uint64_t projection_bytes = (uint64_t)elements * item;
#define KHM_SPLIT_BUFFER(buffer, bytes, name)                                                                               \
    KHM_REQUIRE((buffer).ptr != nullptr && (buffer).len_bytes >= (bytes), "%s buffer holds %llu bytes, needs %llu", name, \
                (unsigned long long)(buffer).len_bytes, (unsigned long long)(bytes))
    KHM_SPLIT_BUFFER(projection, projection_bytes, gated ? "qgkv" : "qkv");
    KHM_SPLIT_BUFFER(q, q_bytes, "q");
    if (gated) KHM_SPLIT_BUFFER(*g, q_bytes, "g");
    KHM_SPLIT_BUFFER(k, kv_bytes, "k");
    KHM_SPLIT_BUFFER(v, kv_bytes, "v");
#undef KHM_SPLIT_BUFFER

    const khm_buffer* all[5] = {&projection, &q, &k, &v, g};
    const uint32_t unit_bytes = unit_bytes_for(head_row_bytes, all, gated ? 5 : 4);
    KHM_REQUIRE(unit_bytes >= item, "%s split buffers must be aligned to their element size", what);
    SplitParams p{};
    p.projection = projection.ptr;
    p.q = q.ptr;
    p.g = gated ? g->ptr : nullptr;
    p.k = k.ptr;
    p.v = v.ptr;
    p.replay_parameters = replay_parameters;
    p.num_active_tokens = DeviceReplayU32{num_active_tokens.is_parameter, num_active_tokens.value};
    p.head_units = (uint32_t)(head_row_bytes / unit_bytes);
    p.q_units = config->num_q_heads * p.head_units;
    p.kv_units = config->num_kv_heads * p.head_units;
    p.row_units = (uint32_t)(row_heads * p.head_units);
    const uint32_t row_blocks = (p.row_units + 255) / 256;
    p.row_blocks = row_blocks;
    const uint64_t blocks = (uint64_t)num_total_tokens * row_blocks;
    KHM_REQUIRE(blocks <= 0x7fffffffull, "%s split needs %llu blocks, more than one launch covers", what, (unsigned long long)blocks);
    const dim3 grid((uint32_t)blocks, 1, 1);
    if (gated) launch_split<true>(unit_bytes, grid, static_cast<hipStream_t>(stream), p);
    else launch_split<false>(unit_bytes, grid, static_cast<hipStream_t>(stream), p);
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "%s split launch failed: %s", what, hipGetErrorString(status));
    return KHM_OK;
}

}  // namespace khm

using namespace khm;

// Config::qgkv_width / qkv_width (qgkv_split.rs:119-133): elements of one token's projection row, 0 if it does not fit.
extern "C" uint64_t khm_gqa_qgkv_width(const khm_gqa_projection_split_config* config) {
    if (config == nullptr) return 0;
    const uint64_t heads = 2ull * config->num_q_heads + 2ull * config->num_kv_heads;
    return heads > 0xffffffffull ? 0 : heads * config->head_dim;
}

extern "C" uint64_t khm_gqa_qkv_width(const khm_gqa_projection_split_config* config) {
    if (config == nullptr) return 0;
    const uint64_t heads = (uint64_t)config->num_q_heads + 2ull * config->num_kv_heads;
    return heads > 0xffffffffull ? 0 : heads * config->head_dim;
}

extern "C" int khm_gqa_qgkv_split(const khm_gqa_projection_split_config* config, uint32_t num_total_tokens, khm_buffer qgkv,
                                  khm_buffer q, khm_buffer g, khm_buffer k, khm_buffer v, khm_replay_u32 num_active_tokens,
                                  const uint32_t* replay_parameters, void* stream) {
    return projection_split(true, config, num_total_tokens, qgkv, q, &g, k, v, num_active_tokens, replay_parameters, stream);
}

extern "C" int khm_gqa_qkv_split(const khm_gqa_projection_split_config* config, uint32_t num_total_tokens, khm_buffer qkv,
                                 khm_buffer q, khm_buffer k, khm_buffer v, khm_replay_u32 num_active_tokens,
                                 const uint32_t* replay_parameters, void* stream) {
    return projection_split(false, config, num_total_tokens, qkv, q, nullptr, k, v, num_active_tokens, replay_parameters, stream);
}
