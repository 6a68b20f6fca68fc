// Per-head RMSNorm followed by rotary position embedding (default or Yarn-scaled): the producer of the SDPA's Q and of
// K before the page write.
//
// Mirrors rms_norm_rope::{Config, RopeScaling, Shape, Buffers, Compute, Invocation}
// (crates/inference-backend-metal/src/components/rms_norm_rope.rs:53-403) and the kernels rms_norm_rope_{f32,bf16}
// [_weight_f32] (.../metal/rms_norm_rope.metal:6-174).  The rotary table (inverse frequencies, at most 128 floats) is
// computed on the host per call and travels as a kernel argument, so nothing is allocated.
#include <hip/hip_runtime.h>

#include <cmath>
#include <vector>

#include "common.h"
#include "device_math.hip.h"
#include "device_params.h"

namespace khm {

constexpr int kMaxRopeHalf = 128;

struct RmsNormRopeParams {
    const void* input;                   // [T][H][D]
    const void* norm_weight;             // [D]
    const uint32_t* flat_token_indices;  // [T]: positions
    void* output;
    const uint32_t* replay_parameters;
    DeviceReplayU32 num_active_tokens;
    uint32_t num_heads;
    uint32_t head_dim;
    uint32_t rope_dim;
    float eps;
    float attention_factor;
    float inverse_frequencies[kMaxRopeHalf];
};

__device__ __forceinline__ float widen(float v) { return v; }
__device__ __forceinline__ float widen(uint16_t v) { return bf16_bits_to_f32(v); }

// apply_norm of rms_norm_rope.metal:6-20: with bf16 input AND bf16 weight both products are rounded to bf16 (the
// reference multiplies bfloat values); every other combination stays in f32.
template <typename T, typename W>
__device__ __forceinline__ float apply_norm(T input, W weight, float inv_rms) {
    if constexpr (sizeof(T) == 2 && sizeof(W) == 2) {
        const float normalized = round_to_bf16(widen(input) * inv_rms);
        return round_to_bf16(widen(weight) * normalized);
    } else {
        return widen(weight) * widen(input) * inv_rms;
    }
}

__device__ __forceinline__ void store_out(float* out, uint64_t index, float v) { out[index] = v; }
__device__ __forceinline__ void store_out(uint16_t* out, uint64_t index, float v) { out[index] = f32_to_bf16_bits(v); }

// One wavefront per (token, head) row.  Lane l sums the squares of elements 4l .. 4l+3 (+256 per round) in order, as a
// thread of the reference does, then the lanes combine.
template <typename T, typename W>
__global__ __launch_bounds__(64) void rms_norm_rope_kernel(const RmsNormRopeParams p) {
    const uint32_t row = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint64_t total_rows = (uint64_t)resolve_u32(p.num_active_tokens, p.replay_parameters) * p.num_heads;
    if (row >= total_rows) return;
    const uint32_t token = row / p.num_heads;
    const uint64_t base = (uint64_t)row * p.head_dim;
    const T* input = static_cast<const T*>(p.input);
    const W* weight = static_cast<const W*>(p.norm_weight);
    T* output = static_cast<T*>(p.output);

    float acc = 0.0f;
    for (uint32_t r = lane * 4; r < p.head_dim; r += 256) {
        for (uint32_t i = 0; i < 4 && r + i < p.head_dim; ++i) {
            const float x = widen(input[base + r + i]);
            acc += x * x;
        }
    }
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1) acc += __shfl_xor(acc, step);
    const float inv_rms = 1.0f / sqrtf(acc / (float)p.head_dim + p.eps);

    const uint32_t rope_half = p.rope_dim / 2;
    const float position = (float)p.flat_token_indices[token];
    for (uint32_t d = lane; d < p.head_dim; d += 64) {
        if (d < rope_half) {
            const uint32_t d2 = d + rope_half;
            const float x1 = apply_norm(input[base + d], weight[d], inv_rms);
            const float x2 = apply_norm(input[base + d2], weight[d2], inv_rms);
            const float theta = position * p.inverse_frequencies[d];
            float s, c;
            sincosf(theta, &s, &c);
            store_out(output, base + d, p.attention_factor * (x1 * c - x2 * s));
            store_out(output, base + d2, p.attention_factor * (x1 * s + x2 * c));
        } else if (d >= p.rope_dim) {
            store_out(output, base + d, apply_norm(input[base + d], weight[d], inv_rms));
        }
    }
}

// Eight consecutive elements of a row as one lane holds them.
template <typename T>
struct Row8;
template <>
struct Row8<float> {
    static __device__ __forceinline__ void load(const float* source, float (&x)[8]) {
        const float4 a = *reinterpret_cast<const float4*>(source), b = *reinterpret_cast<const float4*>(source + 4);
        x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
    }
    static __device__ __forceinline__ void store(float* target, const float (&x)[8]) {
        *reinterpret_cast<float4*>(target) = make_float4(x[0], x[1], x[2], x[3]);
        *reinterpret_cast<float4*>(target + 4) = make_float4(x[4], x[5], x[6], x[7]);
    }
};
template <>
struct Row8<uint16_t> {
    static __device__ __forceinline__ void load(const uint16_t* source, float (&x)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(source);
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) x[2 * i] = __uint_as_float(words[i] << 16), x[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(uint16_t* target, const float (&x)[8]) {
        *reinterpret_cast<uint4*>(target) = make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]), pack_bf16x2(x[6], x[7]));
    }
};

// Lane exchanges that stay in the VALU: DPP inside a 16-lane row, v_permlane{16,32}_swap across rows.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
// The value lane (l ^ 16) holds (ROWS = 16) or lane (l ^ 32) holds (ROWS = 32).
template <int ROWS>
__device__ __forceinline__ float value_of_lane_xor(float v, uint32_t lane) {
    const uint32_t bits = __float_as_uint(v);
    if constexpr (ROWS == 16) {
        const auto halves = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        return __uint_as_float((lane & 16u) ? halves[0] : halves[1]);
    } else {
        const auto halves = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        return __uint_as_float((lane & 32u) ? halves[0] : halves[1]);
    }
}
// Sum over the LPR lanes of a row (8, 16, 32 or 64 aligned lanes), in every lane: quad_perm [1,0,3,2], quad_perm [2,3,0,1],
// row_half_mirror, then row_mirror and the row swaps as far as the row reaches.
template <uint32_t LPR>
__device__ __forceinline__ float sum_in_row(float v, uint32_t lane) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    if constexpr (LPR >= 16) v += dpp_move<0x140>(v);
    if constexpr (LPR >= 32) v += value_of_lane_xor<16>(v, lane);
    if constexpr (LPR == 64) v += value_of_lane_xor<32>(v, lane);
    return v;
}

// The same arithmetic for head_dim <= 512 with head_dim and rope_dim / 2 multiples of 8.  A row occupies LPR = 8, 16, 32
// or 64 lanes (8 elements per lane from one 16- or 32-byte load), so a wavefront holds 64 / LPR rows side by side; the
// rotary partner (rope_dim / 2 elements away) is the same slot of the lane PARTNER = rope_dim / 16 away: 8 lanes is a
// DPP row rotation, 16 and 32 the row swaps, anything else (PARTNER = 0) a generic shuffle.  A block serves the heads
// of ONE token: the first lanes evaluate the token's sines and cosines once into LDS, and each wave issues the loads
// of up to kRowsInFlight row groups before it uses the first.
constexpr int kRowsInFlight = 4;

template <typename T, typename W, uint32_t LPR, uint32_t PARTNER>
__global__ __launch_bounds__(256) void rms_norm_rope_rows_kernel(const RmsNormRopeParams p) {
    constexpr uint32_t kRowsPerWave = 64u / LPR;
    constexpr uint32_t kHeadsPerBlock = 4 * kRowsInFlight * kRowsPerWave;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t token = blockIdx.x;
    if (token >= resolve_u32(p.num_active_tokens, p.replay_parameters)) return;
    const uint32_t sub_row = lane / LPR;
    const uint32_t first = (lane % LPR) * 8;
    const bool holds = first < p.head_dim;
    const uint32_t rope_half = p.rope_dim / 2;
    const bool lower = first < rope_half, rotated = first < p.rope_dim;
    const int partner_lane = ((int)lane + (lower ? (int)(rope_half / 8) : -(int)(rope_half / 8))) & 63;

    float x[kRowsInFlight][8];
    uint32_t heads[kRowsInFlight];
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
        heads[j] = blockIdx.y * kHeadsPerBlock + (j * 4 + wave) * kRowsPerWave + sub_row;
#pragma unroll
        for (int i = 0; i < 8; ++i) x[j][i] = 0.0f;
        if (holds && heads[j] < p.num_heads) Row8<T>::load(static_cast<const T*>(p.input) + ((uint64_t)token * p.num_heads + heads[j]) * p.head_dim + first, x[j]);
    }
    // the token's rotation table, one sine/cosine evaluation per rotary pair for the whole block
    __shared__ __align__(16) float sines[kMaxRopeHalf];
    __shared__ __align__(16) float cosines[kMaxRopeHalf];
    if (threadIdx.x < rope_half) {
        const float position = (float)p.flat_token_indices[token];
        sincosf(position * p.inverse_frequencies[threadIdx.x], &sines[threadIdx.x], &cosines[threadIdx.x]);
    }
    float w[8], sine[8], cosine[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = 0.0f, sine[i] = 0.0f, cosine[i] = 1.0f;
    if (holds) Row8<W>::load(static_cast<const W*>(p.norm_weight) + first, w);
    __syncthreads();
    if (rotated) {
        const uint32_t pair = lower ? first : first - rope_half;
        Row8<float>::load(sines + pair, sine);
        Row8<float>::load(cosines + pair, cosine);
    }
    const float inverse_dim = 1.0f / (float)p.head_dim;
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc += x[j][i] * x[j][i];
        acc = sum_in_row<LPR>(acc, lane);
        // v_rsq_f32 (1 ulp) and one Newton step, which leaves the error below that of a correctly rounded rsqrt's input
        const float mean = acc * inverse_dim + p.eps;
        float inv_rms = __builtin_amdgcn_rsqf(mean);
        inv_rms = inv_rms * __builtin_fmaf(-0.5f * mean * inv_rms, inv_rms, 1.5f);
        float out[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float normed;
            if constexpr (sizeof(T) == 2 && sizeof(W) == 2) {
                normed = round_to_bf16(w[i] * round_to_bf16(x[j][i] * inv_rms));
            } else {
                normed = w[i] * x[j][i] * inv_rms;
            }
            float partner;
            if constexpr (PARTNER == 8) partner = dpp_move<0x128>(normed);          // row_ror:8 = lane ^ 8 inside a 16-lane row
            else if constexpr (PARTNER == 16) partner = value_of_lane_xor<16>(normed, lane);
            else if constexpr (PARTNER == 32) partner = value_of_lane_xor<32>(normed, lane);
            else partner = __shfl(normed, partner_lane);
            out[i] = normed;
            if (rotated) {
                out[i] = lower ? p.attention_factor * (normed * cosine[i] - partner * sine[i])
                               : p.attention_factor * (partner * sine[i] + normed * cosine[i]);
            }
        }
        if (holds && heads[j] < p.num_heads) Row8<T>::store(static_cast<T*>(p.output) + ((uint64_t)token * p.num_heads + heads[j]) * p.head_dim + first, out);
    }
}

// RopeScaling::yarn_kernel_parameters (rms_norm_rope.rs:206-243).
static int yarn_correction_range(const khm_rms_norm_rope_config& config, float* low_out, float* high_out) {
    const khm_rope_scaling& yarn = config.rope_scaling;
    auto correction = [&](float rotations) {
        const double dimension = (double)config.rope_dim;
        const double base = (double)config.rope_theta;
        const double original_length = (double)yarn.original_max_position_embeddings;
        const double tau = 6.283185307179586476925286766559;
        return (float)(dimension * std::log(original_length / ((double)rotations * tau)) / (2.0 * std::log(base)));
    };
    float low = std::fmax(correction(yarn.beta_fast), 0.0f);
    float high = std::fmin(correction(yarn.beta_slow), (float)(config.rope_dim > 0 ? config.rope_dim - 1 : 0));
    if (yarn.truncate) {
        low = std::floor(low);
        high = std::ceil(high);
    }
    KHM_REQUIRE(low <= high, "Yarn correction range must be ordered");
    if (low == high) high += 0.001f;
    *low_out = low;
    *high_out = high;
    return KHM_OK;
}

// Config::validate + RopeScaling::validate (rms_norm_rope.rs:126-204).
static int validate_rms_norm_rope_config(const khm_rms_norm_rope_config* config) {
    KHM_REQUIRE(config != nullptr, "RMSNorm/RoPE config must not be null");
    KHM_REQUIRE(config->num_heads > 0 && config->head_dim > 0 && config->rope_dim > 0, "RMSNorm/RoPE requires heads, a head dimension and a rope dimension");
    KHM_REQUIRE(config->rope_dim <= config->head_dim, "RMSNorm/RoPE rope_dim must not exceed head_dim");
    KHM_REQUIRE(config->rope_dim % 2 == 0, "RMSNorm/RoPE rope_dim must be even");
    KHM_REQUIRE(std::isfinite(config->eps) && config->eps > 0.0f, "RMSNorm/RoPE eps must be finite and positive");
    KHM_REQUIRE(std::isfinite(config->rope_theta) && config->rope_theta > 0.0f, "RMSNorm/RoPE rope_theta must be finite and positive");
    const khm_rope_scaling& s = config->rope_scaling;
    KHM_REQUIRE(s.kind == KHM_ROPE_SCALING_DEFAULT || s.kind == KHM_ROPE_SCALING_YARN, "unknown rope scaling kind");
    if (s.kind == KHM_ROPE_SCALING_YARN) {
        KHM_REQUIRE(std::isfinite(s.factor) && s.factor >= 1.0f, "Yarn factor must be finite and at least 1");
        KHM_REQUIRE(std::isfinite(s.attention_factor) && s.attention_factor > 0.0f, "Yarn attention_factor must be finite and positive");
        KHM_REQUIRE(std::isfinite(s.beta_fast) && s.beta_fast > 0.0f && std::isfinite(s.beta_slow) && s.beta_slow > 0.0f,
                    "Yarn beta_fast and beta_slow must be finite and positive");
        KHM_REQUIRE(s.beta_fast >= s.beta_slow, "Yarn beta_fast must not be below beta_slow");
        KHM_REQUIRE(s.original_max_position_embeddings > 0, "Yarn original_max_position_embeddings must be positive");
        KHM_REQUIRE(config->rope_theta > 1.0f, "Yarn rope_theta must be greater than 1");
    }
    KHM_REQUIRE(config->dtype == KHM_DTYPE_F32 || config->dtype == KHM_DTYPE_BF16, "unsupported RMSNorm/RoPE IO dtype");
    KHM_REQUIRE(config->norm_weight_dtype == KHM_DTYPE_F32 || config->norm_weight_dtype == KHM_DTYPE_BF16, "unsupported RMSNorm/RoPE weight dtype");
    return KHM_OK;
}

// RopeScaling::kernel_parameters (rms_norm_rope.rs:245-270).
static int rope_kernel_parameters(const khm_rms_norm_rope_config& config, float* inverse_frequencies, float* attention_factor) {
    const uint32_t rope_half = config.rope_dim / 2;
    const bool yarn = config.rope_scaling.kind == KHM_ROPE_SCALING_YARN;
    float low = 0.0f, high = 1.0f;
    if (yarn) {
        if (int status = yarn_correction_range(config, &low, &high)) return status;
    }
    for (uint32_t dimension = 0; dimension < rope_half; ++dimension) {
        float inverse_frequency = std::pow(config.rope_theta, -((float)dimension / (float)rope_half));
        if (yarn) {
            float ramp = ((float)dimension - low) / (high - low);
            ramp = ramp < 0.0f ? 0.0f : (ramp > 1.0f ? 1.0f : ramp);
            inverse_frequency *= 1.0f + ramp * (1.0f / config.rope_scaling.factor - 1.0f);
        }
        KHM_REQUIRE(std::isfinite(inverse_frequency) && inverse_frequency > 0.0f, "RMSNorm/RoPE inverse frequency must be finite and positive");
        inverse_frequencies[dimension] = inverse_frequency;
    }
    *attention_factor = yarn ? config.rope_scaling.attention_factor : 1.0f;
    return KHM_OK;
}

}  // namespace khm

using namespace khm;

extern "C" int khm_rms_norm_rope_yarn_correction_range(const khm_rms_norm_rope_config* config, float* low, float* high) {
    clear_error();
    if (int status = validate_rms_norm_rope_config(config)) return status;
    KHM_REQUIRE(low != nullptr && high != nullptr, "low and high must not be null");
    KHM_REQUIRE(config->rope_scaling.kind == KHM_ROPE_SCALING_YARN, "the correction range exists for Yarn scaling only");
    return yarn_correction_range(*config, low, high);
}

extern "C" int khm_rms_norm_rope_kernel_parameters(const khm_rms_norm_rope_config* config, float* inverse_frequencies, uint32_t capacity,
                                                   float* attention_factor) {
    clear_error();
    if (int status = validate_rms_norm_rope_config(config)) return status;
    KHM_REQUIRE(inverse_frequencies != nullptr && attention_factor != nullptr, "outputs must not be null");
    KHM_REQUIRE(capacity >= config->rope_dim / 2, "inverse_frequencies holds %u values, needs %u", capacity, config->rope_dim / 2);
    std::vector<float> table(config->rope_dim / 2);
    if (int status = rope_kernel_parameters(*config, table.data(), attention_factor)) return status;
    for (size_t i = 0; i < table.size(); ++i) inverse_frequencies[i] = table[i];
    return KHM_OK;
}

extern "C" int khm_rms_norm_rope(const khm_rms_norm_rope_config* config, uint32_t num_total_tokens, const khm_rms_norm_rope_buffers* buffers,
                                 khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    if (int status = validate_rms_norm_rope_config(config)) return status;
    KHM_REQUIRE(buffers != nullptr, "buffers must not be null");
    KHM_REQUIRE(config->rope_dim / 2 <= (uint32_t)kMaxRopeHalf, "gfx950 RMSNorm/RoPE holds at most %d rotary pairs", kMaxRopeHalf);
    // Shape::validate (rms_norm_rope.rs:278-284)
    KHM_REQUIRE(num_total_tokens > 0, "RMSNorm/RoPE requires tokens");
    const __uint128_t rows = (__uint128_t)num_total_tokens * config->num_heads;
    KHM_REQUIRE(rows <= 0xffffffffull, "RMSNorm/RoPE token-head rows exceeds the shader u32 count domain");
    KHM_REQUIRE(rows * config->head_dim <= 0xffffffffull, "RMSNorm/RoPE elements exceeds the shader u32 element-index domain");
    // Invocation::validate (rms_norm_rope.rs:386-397)
    if (!num_active_tokens.is_parameter) {
        KHM_REQUIRE(num_active_tokens.value >= 1 && num_active_tokens.value <= num_total_tokens,
                    "num_active_tokens=%u is outside its replay domain [1, %u]", num_active_tokens.value, num_total_tokens);
    } else {
        KHM_REQUIRE(replay_parameters != nullptr, "num_active_tokens is a replay parameter but no parameter block was given");
    }
    const uint64_t bytes = (uint64_t)rows * config->head_dim * dtype_item_size(config->dtype);
    const uint64_t weight_bytes = (uint64_t)config->head_dim * dtype_item_size(config->norm_weight_dtype);
#define KHM_NORM_AT_LEAST(buffer, need, name)                                                                                  \
    KHM_REQUIRE((buffer).ptr != nullptr && (buffer).len_bytes >= (uint64_t)(need), "%s buffer holds %llu bytes, needs %llu", name, \
                (unsigned long long)(buffer).len_bytes, (unsigned long long)(need))
    KHM_NORM_AT_LEAST(buffers->input, bytes, "input");
    KHM_NORM_AT_LEAST(buffers->norm_weight, weight_bytes, "norm_weight");
    KHM_NORM_AT_LEAST(buffers->flat_token_indices, (uint64_t)num_total_tokens * 4, "flat_token_indices");
    KHM_NORM_AT_LEAST(buffers->output, bytes, "output");
#undef KHM_NORM_AT_LEAST

    RmsNormRopeParams p{};
    if (int status = rope_kernel_parameters(*config, p.inverse_frequencies, &p.attention_factor)) return status;
    p.input = buffers->input.ptr;
    p.norm_weight = buffers->norm_weight.ptr;
    p.flat_token_indices = static_cast<const uint32_t*>(buffers->flat_token_indices.ptr);
    p.output = buffers->output.ptr;
    p.replay_parameters = replay_parameters;
    p.num_active_tokens = DeviceReplayU32{num_active_tokens.is_parameter, num_active_tokens.value};
    p.num_heads = config->num_heads;
    p.head_dim = config->head_dim;
    p.rope_dim = config->rope_dim;
    p.eps = config->eps;
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    const bool io_bf16 = config->dtype == KHM_DTYPE_BF16, weight_bf16 = config->norm_weight_dtype == KHM_DTYPE_BF16;
    // vector loads need 16-byte aligned rows; allocator-aligned bases and head_dim % 8 == 0 give that
    const bool aligned = ((uintptr_t)p.input | (uintptr_t)p.output | (uintptr_t)p.norm_weight) % 16 == 0;
    if (aligned && config->head_dim <= 512 && config->head_dim % 8 == 0 && (config->rope_dim / 2) % 8 == 0) {
        const uint32_t lanes_per_row = config->head_dim <= 64 ? 8u : (config->head_dim <= 128 ? 16u : (config->head_dim <= 256 ? 32u : 64u));
        const uint32_t heads_per_block = 4 * kRowsInFlight * (64u / lanes_per_row);
        const dim3 grid(num_total_tokens, (config->num_heads + heads_per_block - 1) / heads_per_block);
        const uint32_t partner_distance = config->rope_dim / 16;   // lanes between the halves of a rotary pair
        const bool vector_partner = partner_distance == 8 || partner_distance == 16 || partner_distance == 32;
        const uint32_t partner = vector_partner && partner_distance < lanes_per_row ? partner_distance : 0;
        auto launch = [&](auto io_tag, auto weight_tag) {
            typedef decltype(io_tag) T;
            typedef decltype(weight_tag) W;
#define KHM_ROWS_CASE(LPR, PARTNER)                                                                                        \
    if (lanes_per_row == LPR && partner == PARTNER) {                                                                      \
        hipLaunchKernelGGL((rms_norm_rope_rows_kernel<T, W, LPR, PARTNER>), grid, dim3(256), 0, hip_stream, p);             \
        return;                                                                                                            \
    }
            KHM_ROWS_CASE(8, 0) KHM_ROWS_CASE(16, 0) KHM_ROWS_CASE(16, 8) KHM_ROWS_CASE(32, 0) KHM_ROWS_CASE(32, 8) KHM_ROWS_CASE(32, 16)
            KHM_ROWS_CASE(64, 0) KHM_ROWS_CASE(64, 8) KHM_ROWS_CASE(64, 16) KHM_ROWS_CASE(64, 32)
#undef KHM_ROWS_CASE
        };
        if (io_bf16 && weight_bf16) launch(uint16_t{}, uint16_t{});
        else if (io_bf16) launch(uint16_t{}, float{});
        else if (weight_bf16) launch(float{}, uint16_t{});
        else launch(float{}, float{});
    } else {
        const dim3 grid((uint32_t)rows);
        if (io_bf16 && weight_bf16) hipLaunchKernelGGL((rms_norm_rope_kernel<uint16_t, uint16_t>), grid, dim3(64), 0, hip_stream, p);
        else if (io_bf16) hipLaunchKernelGGL((rms_norm_rope_kernel<uint16_t, float>), grid, dim3(64), 0, hip_stream, p);
        else if (weight_bf16) hipLaunchKernelGGL((rms_norm_rope_kernel<float, uint16_t>), grid, dim3(64), 0, hip_stream, p);
        else hipLaunchKernelGGL((rms_norm_rope_kernel<float, float>), grid, dim3(64), 0, hip_stream, p);
    }
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "RMSNorm/RoPE launch failed: %s", hipGetErrorString(status));
    return KHM_OK;
}
