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

template <typename T>
struct Row4;
template <>
struct Row4<float> {
    using Vec = float4;
    static __device__ __forceinline__ void unpack(const Vec& v, float (&x)[4]) { x[0] = v.x, x[1] = v.y, x[2] = v.z, x[3] = v.w; }
    static __device__ __forceinline__ Vec pack(const float (&x)[4]) { return make_float4(x[0], x[1], x[2], x[3]); }
};
template <>
struct Row4<uint16_t> {
    using Vec = uint2;
    static __device__ __forceinline__ void unpack(const Vec& v, float (&x)[4]) {
        x[0] = bf16_bits_to_f32((uint16_t)(v.x & 0xffffu)), x[1] = bf16_bits_to_f32((uint16_t)(v.x >> 16));
        x[2] = bf16_bits_to_f32((uint16_t)(v.y & 0xffffu)), x[3] = bf16_bits_to_f32((uint16_t)(v.y >> 16));
    }
    static __device__ __forceinline__ Vec pack(const float (&x)[4]) {
        return make_uint2((uint32_t)f32_to_bf16_bits(x[0]) | ((uint32_t)f32_to_bf16_bits(x[1]) << 16),
                          (uint32_t)f32_to_bf16_bits(x[2]) | ((uint32_t)f32_to_bf16_bits(x[3]) << 16));
    }
};

// Lane exchanges that stay in the VALU: DPP inside a 16-lane row, v_permlane{16,32}_swap across rows.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
// Sum over the 16 lanes of a row, in every lane: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror.
__device__ __forceinline__ float sum_in_row16(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    return v;
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

// The same arithmetic for head_dim <= 256 with head_dim and rope_dim / 2 multiples of 4.  A row occupies
// LPR = 16, 32 or 64 lanes (4 elements per lane from one vector load), so a wavefront holds 64 / LPR rows side by side;
// the rotary partner (rope_dim / 2 elements away) is the same slot of the lane rope_dim / 8 away.  A block serves up
// to 16 * 64 / LPR heads of ONE token: each lane evaluates the token's sines and cosines once and reuses them for the
// kRowsInFlight rows it visits, whose loads are all issued before the first is used.
constexpr int kRowsInFlight = 8;

// LPR (lanes per row) and PARTNER (lanes between an element and its rotary partner: 16 or 32 for the VALU swaps, 0 for
// any other distance through a generic shuffle) are compile-time, so the row loop is straight-line code.
template <typename T, typename W, uint32_t LPR, uint32_t PARTNER>
__global__ __launch_bounds__(256) void rms_norm_rope_rows_kernel(const RmsNormRopeParams p) {
    constexpr uint32_t lanes_per_row = LPR;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t token = blockIdx.x;
    if (token >= resolve_u32(p.num_active_tokens, p.replay_parameters)) return;
    const uint32_t rows_per_wave = 64u / lanes_per_row;
    const uint32_t sub_row = lane / lanes_per_row;
    const uint32_t first = (lane % lanes_per_row) * 4;
    const bool holds = first < p.head_dim;
    const uint32_t rope_half = p.rope_dim / 2;
    const bool lower = first < rope_half, rotated = first < p.rope_dim;
    const int partner_lane = ((int)lane + (lower ? (int)(rope_half / 4) : -(int)(rope_half / 4))) & 63;

    using Vec = typename Row4<T>::Vec;
    const uint32_t heads_per_block = 4 * kRowsInFlight * rows_per_wave;
    Vec raw[kRowsInFlight];
    uint32_t heads[kRowsInFlight];
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
        heads[j] = blockIdx.y * heads_per_block + (j * 4 + wave) * rows_per_wave + sub_row;
        raw[j] = Vec{};
        if (holds && heads[j] < p.num_heads) {
            raw[j] = *reinterpret_cast<const Vec*>(static_cast<const T*>(p.input) + ((uint64_t)token * p.num_heads + heads[j]) * p.head_dim + first);
        }
    }
    // the token's rotation table, one sine/cosine evaluation per rotary pair for the whole block
    __shared__ __align__(16) float sines[kMaxRopeHalf];
    __shared__ __align__(16) float cosines[kMaxRopeHalf];
    if (threadIdx.x < rope_half) {
        const float position = (float)p.flat_token_indices[token];
        sincosf(position * p.inverse_frequencies[threadIdx.x], &sines[threadIdx.x], &cosines[threadIdx.x]);
    }
    float w[4] = {0.0f, 0.0f, 0.0f, 0.0f}, sine[4] = {0.0f, 0.0f, 0.0f, 0.0f}, cosine[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (holds) Row4<W>::unpack(*reinterpret_cast<const typename Row4<W>::Vec*>(static_cast<const W*>(p.norm_weight) + first), w);
    __syncthreads();
    if (rotated) {
        const uint32_t pair = lower ? first : first - rope_half;
        Row4<float>::unpack(*reinterpret_cast<const float4*>(sines + pair), sine);
        Row4<float>::unpack(*reinterpret_cast<const float4*>(cosines + pair), cosine);
    }
    const float inverse_dim = 1.0f / (float)p.head_dim;
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
        float x[4];
        Row4<T>::unpack(raw[j], x);
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc += x[i] * x[i];
        acc = sum_in_row16(acc);
        if constexpr (LPR >= 32) acc += value_of_lane_xor<16>(acc, lane);
        if constexpr (LPR == 64) acc += value_of_lane_xor<32>(acc, lane);
        // v_rsq_f32 (1 ulp) and one Newton step, which leaves the error below that of a correctly rounded rsqrt's input
        const float mean = acc * inverse_dim + p.eps;
        float inv_rms = __builtin_amdgcn_rsqf(mean);
        inv_rms = inv_rms * __builtin_fmaf(-0.5f * mean * inv_rms, inv_rms, 1.5f);
        float out[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float normed;
            if constexpr (sizeof(T) == 2 && sizeof(W) == 2) {
                normed = round_to_bf16(w[i] * round_to_bf16(x[i] * inv_rms));
            } else {
                normed = w[i] * x[i] * inv_rms;
            }
            float partner;
            if constexpr (PARTNER == 16) partner = value_of_lane_xor<16>(normed, lane);
            else if constexpr (PARTNER == 32) partner = value_of_lane_xor<32>(normed, lane);
            else partner = __shfl(normed, partner_lane);
            out[i] = normed;
            if (rotated) {
                out[i] = lower ? p.attention_factor * (normed * cosine[i] - partner * sine[i])
                               : p.attention_factor * (partner * sine[i] + normed * cosine[i]);
            }
        }
        if (holds && heads[j] < p.num_heads) {
            *reinterpret_cast<Vec*>(static_cast<T*>(p.output) + ((uint64_t)token * p.num_heads + heads[j]) * p.head_dim + first) = Row4<T>::pack(out);
        }
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
    // vector loads need 16-byte (f32) / 8-byte (bf16) aligned rows; cudaMalloc-style bases and head_dim % 4 == 0 give that
    const bool aligned = ((uintptr_t)p.input | (uintptr_t)p.output | (uintptr_t)p.norm_weight) % 16 == 0;
    if (aligned && config->head_dim <= 256 && config->head_dim % 4 == 0 && (config->rope_dim / 2) % 4 == 0) {
        const uint32_t lanes_per_row = config->head_dim <= 64 ? 16u : (config->head_dim <= 128 ? 32u : 64u);
        const uint32_t heads_per_block = 4 * kRowsInFlight * (64u / lanes_per_row);
        const dim3 grid(num_total_tokens, (config->num_heads + heads_per_block - 1) / heads_per_block);
        const uint32_t partner_distance = config->rope_dim / 8;   // lanes between the halves of a rotary pair
        const uint32_t partner = partner_distance == 16 || partner_distance == 32 ? partner_distance : 0;
        auto launch = [&](auto io_tag, auto weight_tag) {
            typedef decltype(io_tag) T;
            typedef decltype(weight_tag) W;
#define KHM_ROWS_CASE(LPR, PARTNER)                                                                                        \
    if (lanes_per_row == LPR && partner == PARTNER) {                                                                      \
        hipLaunchKernelGGL((rms_norm_rope_rows_kernel<T, W, LPR, PARTNER>), grid, dim3(256), 0, hip_stream, p);             \
        return;                                                                                                            \
    }
            KHM_ROWS_CASE(16, 0) KHM_ROWS_CASE(32, 0) KHM_ROWS_CASE(32, 16) KHM_ROWS_CASE(64, 0) KHM_ROWS_CASE(64, 16) KHM_ROWS_CASE(64, 32)
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
