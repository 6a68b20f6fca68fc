// Per-head RMSNorm followed by rotary position embedding (default or Yarn-scaled): the producer of the SDPA's Q and of
// K before the page write.
//
// Mirrors rms_norm_rope::{Config, RopeScaling, Shape, Buffers, Compute, Invocation}
// (crates/inference-backend-metal/src/components/rms_norm_rope.rs:53-403) and the kernels rms_norm_rope_{f32,bf16}
// [_weight_f32] (.../metal/rms_norm_rope.metal:6-174).  The rotary table (inverse frequencies, at most 128 floats) is
// computed on the host per call and travels as a kernel argument, so nothing is allocated.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <type_traits>
#include <vector>

#include "common.h"
#include "device_math.hip.h"
#include "device_params.h"
#include "fp8_device.hip.h"
#include "page_write_params.h"

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
    uint32_t tokens_per_block;      // rows kernels: tokens a block serves (more than one when there are few heads)
    uint32_t row_slots_per_token_shift;  // rows kernels: log2 of the row slots of a block that one token takes
    uint32_t input_row_stride;      // rows kernels: elements from a token's first input row to the next token's (H * D when packed)
    uint32_t input_head_stride;     // rows kernels: elements from a head's input row to the next head's (D when packed)
    void* gate_output;              // projection rows kernel: [T][H][D] rows copied from the D elements behind each input row
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
    struct Raw { float4 a, b; };
    static __device__ __forceinline__ Raw zero() { return Raw{make_float4(0.f, 0.f, 0.f, 0.f), make_float4(0.f, 0.f, 0.f, 0.f)}; }
    static __device__ __forceinline__ Raw load_raw(const float* source) {
        return Raw{*reinterpret_cast<const float4*>(source), *reinterpret_cast<const float4*>(source + 4)};
    }
    static __device__ __forceinline__ void unpack(const Raw& raw, float (&x)[8]) {
        x[0] = raw.a.x, x[1] = raw.a.y, x[2] = raw.a.z, x[3] = raw.a.w, x[4] = raw.b.x, x[5] = raw.b.y, x[6] = raw.b.z, x[7] = raw.b.w;
    }
    static __device__ __forceinline__ void load(const float* source, float (&x)[8]) {
        const float4 a = *reinterpret_cast<const float4*>(source), b = *reinterpret_cast<const float4*>(source + 4);
        x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
    }
    static __device__ __forceinline__ void store(float* target, const float (&x)[8]) {
        typedef float F32x4 __attribute__((ext_vector_type(4)));
        const F32x4 low = {x[0], x[1], x[2], x[3]}, high = {x[4], x[5], x[6], x[7]};
        __builtin_nontemporal_store(low, reinterpret_cast<F32x4*>(target));
        __builtin_nontemporal_store(high, reinterpret_cast<F32x4*>(target + 4));
    }
};
template <>
struct Row8<uint16_t> {
    typedef uint4 Raw;
    static __device__ __forceinline__ Raw zero() { return make_uint4(0u, 0u, 0u, 0u); }
    static __device__ __forceinline__ Raw load_raw(const uint16_t* source) { return *reinterpret_cast<const uint4*>(source); }
    static __device__ __forceinline__ void unpack(const Raw& v, float (&x)[8]) {
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) x[2 * i] = __uint_as_float(words[i] << 16), x[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
    }
    static __device__ __forceinline__ void load(const uint16_t* source, float (&x)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(source);
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) x[2 * i] = __uint_as_float(words[i] << 16), x[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(uint16_t* target, const float (&x)[8]) {
        typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
        const U32x4 packed = {pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]), pack_bf16x2(x[6], x[7])};
        __builtin_nontemporal_store(packed, reinterpret_cast<U32x4*>(target));   // written once, read by a later launch
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
constexpr int kPageRowsInFlight = 2;   // the fused page writer: 64 instead of 90 registers, eight waves per SIMD, twice the blocks
constexpr int kMaxTokensPerBlock = 16;

// PAGES: 0 writes the rows to p.output; 1 / 2 scatter them, as K rows, straight into bf16 / FP8 E4M3FN pages through
// the page table and copy the V rows of the same (token, KV head) beside them: RMSNorm + RoPE of K and the K/V page write
// in one pass, the bf16 value the two-kernel sequence would have stored in between being the one that is encoded.
// What differs between the row sets one launch can serve (Q rows to an output buffer, K rows to pages); the rotation
// table, positions and active count are shared (RmsNormRopeParams).
struct RowsRole {
    const void* input;           // first element of token 0, head 0
    const void* norm_weight;     // [D]
    void* output;                // PAGES == 0: [T][H][D]
    void* gate_output;           // GATE: [T][H][D]
    uint32_t num_heads;
    uint32_t input_row_stride;   // elements
    uint32_t input_head_stride;  // elements
    uint32_t v_row_stride;       // PAGES != 0: elements from a token's V rows to the next token's (heads are D apart)
    float eps;
    uint32_t tokens_per_block;
    uint32_t row_slots_per_token_shift;
};
__device__ __forceinline__ RowsRole role_of(const RmsNormRopeParams& p) {
    return RowsRole{p.input, p.norm_weight, p.output, p.gate_output, p.num_heads, p.input_row_stride, p.input_head_stride,
                    p.num_heads * p.head_dim, p.eps, p.tokens_per_block, p.row_slots_per_token_shift};
}

// GATE: the D elements behind every input row (the gate half of a gated projection's head pair) are copied to
// role.gate_output as they are.  `sines` / `cosines` are the block's LDS tables, [kMaxTokensPerBlock * kMaxRopeHalf] each.
template <typename T, typename W, uint32_t LPR, uint32_t PARTNER, int PAGES, bool GATE>
__device__ __forceinline__ void rms_norm_rope_rows(const RmsNormRopeParams& p, const RowsRole& role, const PageWriteParams* pages,
                                                   uint32_t block_x, uint32_t block_y, float* sines, float* cosines) {
    static_assert(PAGES == 0 || sizeof(T) == 2, "pages are written from bf16 rows");
    static_assert(!GATE || (PAGES == 0 && sizeof(T) == 2), "gate rows are copied beside bf16 output rows");
    constexpr uint32_t kRowsPerWave = 64u / LPR;
    constexpr int kRows = PAGES != 0 ? kPageRowsInFlight : kRowsInFlight;   // row groups of a wave
    constexpr uint32_t kRowSlots = 4 * kRows * kRowsPerWave;   // (token, head) rows a block holds
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    // Row slot s of the block belongs to token s >> shift of the block's tokens and to head s & (2^shift - 1) of this
    // block's head group: one token per block when the heads fill the slots, several when there are few heads (the K
    // rows of a grouped-query model), so that every wave has rows and a token's sines and cosines are shared by its heads.
    const uint32_t tokens_per_block = role.tokens_per_block, slot_shift = role.row_slots_per_token_shift;
    const uint32_t num_active_tokens = resolve_u32(p.num_active_tokens, p.replay_parameters);
    const uint32_t first_token = block_x * tokens_per_block;
    if (first_token >= num_active_tokens) return;
    const uint32_t sub_row = lane / LPR;
    const uint32_t first = (lane % LPR) * 8;
    const bool holds = first < p.head_dim;
    const uint32_t rope_half = p.rope_dim / 2;
    const bool lower = first < rope_half, rotated = first < p.rope_dim;
    const int partner_lane = ((int)lane + (lower ? (int)(rope_half / 8) : -(int)(rope_half / 8))) & 63;

    typename Row8<T>::Raw raw[kRows];   // rows stay as loaded until their turn: half the registers of eight floats
    typename Row8<T>::Raw gate_raw[GATE ? kRows : 1];
    uint32_t heads[kRows], tokens[kRows], local_tokens[kRows];
    bool valid[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j) {
        const uint32_t slot = (j * 4 + wave) * kRowsPerWave + sub_row;
        local_tokens[j] = slot >> slot_shift;
        tokens[j] = first_token + local_tokens[j];
        heads[j] = block_y * kRowSlots + (slot & ((1u << slot_shift) - 1u));
        valid[j] = holds && heads[j] < role.num_heads && local_tokens[j] < tokens_per_block && tokens[j] < num_active_tokens;
        raw[j] = Row8<T>::zero();
        const T* source = static_cast<const T*>(role.input) + (uint64_t)tokens[j] * role.input_row_stride + (uint64_t)heads[j] * role.input_head_stride + first;
        if (valid[j]) raw[j] = Row8<T>::load_raw(source);
        if constexpr (GATE) {
            if (valid[j]) gate_raw[j] = Row8<T>::load_raw(source + p.head_dim);
        }
    }
    // Page writes: the V chunks and the page-table walk (request slot, position -> page id) of every row are requested
    // here, beside the K rows, so that their round trips pass under the sine/cosine evaluation and the block barrier
    // instead of standing between the last arithmetic and the stores.
    uint4 v_chunk[PAGES != 0 ? kRows : 1];
    PageTarget target[PAGES != 0 ? kRows : 1];
    if constexpr (PAGES != 0) {
        constexpr uint32_t kElementBytes = PAGES == 2 ? 1 : 2;
        const uint32_t layer = resolve_u32(pages->layer_index, pages->replay_parameters);
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
            v_chunk[j] = make_uint4(0, 0, 0, 0);
            target[j] = PageTarget{0, 0};
            if (valid[j]) {
                v_chunk[j] = *reinterpret_cast<const uint4*>(pages->flat_v + (uint64_t)tokens[j] * role.v_row_stride + heads[j] * p.head_dim + first);
                target[j] = page_target_of(*pages, pages->req_slots[tokens[j]], pages->flat_token_indices[tokens[j]], layer, heads[j], first,
                                           kElementBytes);
            }
        }
    }
    // the rotation tables of the block's tokens, one sine/cosine evaluation per token and rotary pair
    for (uint32_t entry = threadIdx.x; entry < tokens_per_block * rope_half; entry += 256) {
        const uint32_t local = entry / rope_half, pair = entry - local * rope_half;
        if (first_token + local < num_active_tokens) {
            const float position = (float)p.flat_token_indices[first_token + local];
            sincosf(position * p.inverse_frequencies[pair], &sines[local * rope_half + pair], &cosines[local * rope_half + pair]);
        }
    }
    typename Row8<W>::Raw w_raw = Row8<W>::zero();
    if (holds) w_raw = Row8<W>::load_raw(static_cast<const W*>(role.norm_weight) + first);
    __syncthreads();
    if constexpr (GATE) {   // the gate rows have arrived with the input rows: pass them on before the arithmetic
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
            if (valid[j]) store_streaming(static_cast<T*>(role.gate_output) + ((uint64_t)tokens[j] * role.num_heads + heads[j]) * p.head_dim + first, gate_raw[j]);
        }
    }
    const float inverse_dim = 1.0f / (float)p.head_dim;
    float sine[8], cosine[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sine[i] = 0.0f, cosine[i] = 1.0f;
#pragma unroll
    for (int j = 0; j < kRows; ++j) {
        float x[8], w[8];
        Row8<T>::unpack(raw[j], x);
        Row8<W>::unpack(w_raw, w);
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc += x[i] * x[i];
        acc = sum_in_row<LPR>(acc, lane);
        // v_rsq_f32 (1 ulp) and one Newton step, which leaves the error below that of a correctly rounded rsqrt's input
        const float mean = acc * inverse_dim + role.eps;
        float inv_rms = __builtin_amdgcn_rsqf(mean);
        inv_rms = inv_rms * __builtin_fmaf(-0.5f * mean * inv_rms, inv_rms, 1.5f);
        if (rotated && valid[j] && (j == 0 || tokens_per_block > 1)) {   // one token per block: every row shares the first load
            const uint32_t pair = local_tokens[j] * rope_half + (lower ? first : first - rope_half);
            Row8<float>::load(sines + pair, sine);
            Row8<float>::load(cosines + pair, cosine);
        }
        float out[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float normed;
            if constexpr (sizeof(T) == 2 && sizeof(W) == 2) {
                normed = round_to_bf16(w[i] * round_to_bf16(x[i] * inv_rms));
            } else {
                normed = w[i] * x[i] * inv_rms;
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
        if (!valid[j]) continue;
        if constexpr (PAGES == 0) {
            Row8<T>::store(static_cast<T*>(role.output) + ((uint64_t)tokens[j] * role.num_heads + heads[j]) * p.head_dim + first, out);
        } else {
            const uint4 k_chunk = make_uint4(pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3]), pack_bf16x2(out[4], out[5]), pack_bf16x2(out[6], out[7]));
            uint8_t* k_target = pages->pages + target[j].k_offset;
            if constexpr (PAGES == 2) {
                auto encode8 = [](uint4 bits) { return bf16x8_bits_to_fp8x8_e4m3fn(bits); };
                store_streaming(k_target, encode8(k_chunk));
                store_streaming(k_target + target[j].v_distance, encode8(v_chunk[j]));
            } else {
                store_streaming(k_target, k_chunk);
                store_streaming(k_target + target[j].v_distance, v_chunk[j]);
            }
        }
    }
}

#define KHM_ROTATION_TABLES                                                          \
    __shared__ __align__(16) float sines[kMaxTokensPerBlock * kMaxRopeHalf];         \
    __shared__ __align__(16) float cosines[kMaxTokensPerBlock * kMaxRopeHalf]

template <typename T, typename W, uint32_t LPR, uint32_t PARTNER>
__global__ __launch_bounds__(256) void rms_norm_rope_rows_kernel(const RmsNormRopeParams p) {
    KHM_ROTATION_TABLES;
    rms_norm_rope_rows<T, W, LPR, PARTNER, 0, false>(p, role_of(p), nullptr, blockIdx.x, blockIdx.y, sines, cosines);
}

template <typename W, uint32_t LPR, uint32_t PARTNER, bool FP8_PAGES>
__global__ __launch_bounds__(256) void k_norm_rope_page_write_kernel(const RmsNormRopeParams p, const PageWriteParams pages) {
    KHM_ROTATION_TABLES;
    rms_norm_rope_rows<uint16_t, W, LPR, PARTNER, FP8_PAGES ? 2 : 1, false>(p, role_of(p), &pages, blockIdx.x, blockIdx.y, sines, cosines);
}

// Everything between the input projection and the SDPA in one launch (the reference records qgkv_split, q_norm_rope,
// k_norm_rope and kv_page_write: crates/inference-executor-metal/src/attn/gqa/backend.rs:358-412).  The first
// q_blocks blocks take the Q rows straight from the projection rows (head pairs [q | gate] when GATED, gate halves copied
// to their own buffer on the way), the others the K rows and, beside them, the V rows into the pages.  `p` describes the
// Q rows; the K rows differ in what `k_role` holds.
struct ProjectionBlocks {
    uint32_t q_blocks;     // blocks of the Q role, laid out [head group][token group]
    uint32_t q_blocks_x;   // token groups of the Q role
    uint32_t k_blocks_x;   // token groups of the K role
};
template <typename W, uint32_t LPR, uint32_t PARTNER, bool FP8_PAGES, bool GATED>
__global__ __launch_bounds__(256) void projection_norm_rope_page_write_kernel(const RmsNormRopeParams p, const RowsRole k_role,
                                                                              const PageWriteParams pages, const ProjectionBlocks blocks) {
    KHM_ROTATION_TABLES;
    if (blockIdx.x < blocks.q_blocks) {
        const uint32_t block_y = blockIdx.x / blocks.q_blocks_x;
        rms_norm_rope_rows<uint16_t, W, LPR, PARTNER, 0, GATED>(p, role_of(p), nullptr, blockIdx.x - block_y * blocks.q_blocks_x, block_y, sines, cosines);
    } else {
        const uint32_t index = blockIdx.x - blocks.q_blocks;
        const uint32_t block_y = index / blocks.k_blocks_x;
        rms_norm_rope_rows<uint16_t, W, LPR, PARTNER, FP8_PAGES ? 2 : 1, false>(p, k_role, &pages, index - block_y * blocks.k_blocks_x, block_y, sines, cosines);
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

// Config / Shape / Invocation validation of one RMSNorm/RoPE call and its kernel arguments; `output` may be absent when
// the rows go elsewhere (the fused page write).
static int fill_rms_norm_rope_params(const khm_rms_norm_rope_config* config, uint32_t num_total_tokens, const khm_buffer& input,
                                     const khm_buffer& norm_weight, const khm_buffer& flat_token_indices, const khm_buffer* output,
                                     khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, RmsNormRopeParams* out) {
    if (int status = validate_rms_norm_rope_config(config)) return status;
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
    KHM_NORM_AT_LEAST(input, bytes, "input");
    KHM_NORM_AT_LEAST(norm_weight, weight_bytes, "norm_weight");
    KHM_NORM_AT_LEAST(flat_token_indices, (uint64_t)num_total_tokens * 4, "flat_token_indices");
    if (output != nullptr) KHM_NORM_AT_LEAST(*output, bytes, "output");
#undef KHM_NORM_AT_LEAST

    RmsNormRopeParams p{};
    if (int status = rope_kernel_parameters(*config, p.inverse_frequencies, &p.attention_factor)) return status;
    p.input = input.ptr;
    p.norm_weight = norm_weight.ptr;
    p.flat_token_indices = static_cast<const uint32_t*>(flat_token_indices.ptr);
    p.output = output != nullptr ? output->ptr : nullptr;
    p.replay_parameters = replay_parameters;
    p.num_active_tokens = DeviceReplayU32{num_active_tokens.is_parameter, num_active_tokens.value};
    p.num_heads = config->num_heads;
    p.head_dim = config->head_dim;
    p.rope_dim = config->rope_dim;
    p.eps = config->eps;
    p.input_row_stride = config->num_heads * config->head_dim;
    p.input_head_stride = config->head_dim;
    p.gate_output = nullptr;
    *out = p;
    return KHM_OK;
}

// Launch geometry of the rows kernels: lanes per row, the lane distance of a rotary pair when a vector exchange reaches
// it (0 otherwise), and the grid (one block per token and group of heads).
struct RowsGeometry {
    bool fits;   // vector loads need 16-byte aligned rows; head_dim <= 512, head_dim and rope_dim / 2 multiples of 8
    uint32_t lanes_per_row, partner, tokens_per_block, slot_shift;
    dim3 grid;
};
static RowsGeometry rows_geometry(const khm_rms_norm_rope_config& config, uint32_t num_total_tokens, uintptr_t address_bits, int rows_in_flight = kRowsInFlight) {
    RowsGeometry g{};
    g.fits = address_bits % 16 == 0 && config.head_dim <= 512 && config.head_dim % 8 == 0 && (config.rope_dim / 2) % 8 == 0;
    g.lanes_per_row = config.head_dim <= 64 ? 8u : (config.head_dim <= 128 ? 16u : (config.head_dim <= 256 ? 32u : 64u));
    const uint32_t row_slots = 4 * (uint32_t)rows_in_flight * (64u / g.lanes_per_row);   // a power of two
    // few heads: a token takes the next power of two of row slots and a block serves several tokens
    uint32_t slots_per_token = 1;
    while (slots_per_token < config.num_heads && slots_per_token < row_slots) slots_per_token *= 2;
    g.tokens_per_block = std::min<uint32_t>(row_slots / slots_per_token, (uint32_t)kMaxTokensPerBlock);
    g.slot_shift = 0;
    while ((1u << g.slot_shift) < slots_per_token) ++g.slot_shift;
    g.grid = dim3((num_total_tokens + g.tokens_per_block - 1) / g.tokens_per_block, (config.num_heads + row_slots - 1) / row_slots);
    const uint32_t partner_distance = config.rope_dim / 16;   // lanes between the halves of a rotary pair
    const bool vector_partner = partner_distance == 8 || partner_distance == 16 || partner_distance == 32;
    g.partner = vector_partner && partner_distance < g.lanes_per_row ? partner_distance : 0;
    return g;
}

#define KHM_ROWS_CASES(CASE) \
    CASE(8, 0) CASE(16, 0) CASE(16, 8) CASE(32, 0) CASE(32, 8) CASE(32, 16) CASE(64, 0) CASE(64, 8) CASE(64, 16) CASE(64, 32)

extern "C" int khm_rms_norm_rope(const khm_rms_norm_rope_config* config, uint32_t num_total_tokens, const khm_rms_norm_rope_buffers* buffers,
                                 khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(buffers != nullptr, "buffers must not be null");
    RmsNormRopeParams p{};
    if (int status = fill_rms_norm_rope_params(config, num_total_tokens, buffers->input, buffers->norm_weight, buffers->flat_token_indices,
                                               &buffers->output, num_active_tokens, replay_parameters, &p))
        return status;
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    const bool io_bf16 = config->dtype == KHM_DTYPE_BF16, weight_bf16 = config->norm_weight_dtype == KHM_DTYPE_BF16;
    const RowsGeometry geometry = rows_geometry(*config, num_total_tokens, (uintptr_t)p.input | (uintptr_t)p.output | (uintptr_t)p.norm_weight);
    p.tokens_per_block = geometry.tokens_per_block;
    p.row_slots_per_token_shift = geometry.slot_shift;
    if (geometry.fits) {
        auto launch = [&](auto io_tag, auto weight_tag) {
            typedef decltype(io_tag) T;
            typedef decltype(weight_tag) W;
#define KHM_ROWS_CASE(LPR, PARTNER)                                                                                        \
    if (geometry.lanes_per_row == LPR && geometry.partner == PARTNER) {                                                    \
        KHM_LAUNCH((rms_norm_rope_rows_kernel<T, W, LPR, PARTNER>), geometry.grid, dim3(256), 0, hip_stream, p);    \
        return;                                                                                                            \
    }
            KHM_ROWS_CASES(KHM_ROWS_CASE)
#undef KHM_ROWS_CASE
        };
        if (io_bf16 && weight_bf16) launch(uint16_t{}, uint16_t{});
        else if (io_bf16) launch(uint16_t{}, float{});
        else if (weight_bf16) launch(float{}, uint16_t{});
        else launch(float{}, float{});
    } else {
        const dim3 grid(num_total_tokens * config->num_heads);
        if (io_bf16 && weight_bf16) KHM_LAUNCH((rms_norm_rope_kernel<uint16_t, uint16_t>), grid, dim3(64), 0, hip_stream, p);
        else if (io_bf16) KHM_LAUNCH((rms_norm_rope_kernel<uint16_t, float>), grid, dim3(64), 0, hip_stream, p);
        else if (weight_bf16) KHM_LAUNCH((rms_norm_rope_kernel<float, uint16_t>), grid, dim3(64), 0, hip_stream, p);
        else KHM_LAUNCH((rms_norm_rope_kernel<float, float>), grid, dim3(64), 0, hip_stream, p);
    }
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "RMSNorm/RoPE launch failed: %s", hipGetErrorString(status));
    return KHM_OK;
}

// K RMSNorm + RoPE and the K/V page write in one launch (the reference records k_norm_rope -> scratch.k_norm_rope ->
// kv_page_write: crates/inference-executor-metal/src/attn/gqa/backend.rs:382-412): the normalized, rotated K row is
// rounded to bf16 exactly as the first kernel would store it and goes straight into its page, V is copied beside it.
extern "C" int khm_k_norm_rope_page_write(const khm_rms_norm_rope_config* norm_config, const khm_kv_page_write_config* page_config,
                                          const khm_kv_page_write_shape* shape, const khm_k_norm_rope_page_write_buffers* buffers,
                                          khm_replay_u32 num_active_tokens, khm_replay_u32 page_table_index,
                                          const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(norm_config != nullptr && page_config != nullptr && shape != nullptr && buffers != nullptr,
                "configs, shape and buffers must not be null");
    KHM_REQUIRE(norm_config->num_heads == page_config->num_kv_heads && norm_config->head_dim == page_config->head_dim,
                "K RMSNorm/RoPE rows [%u][%u] do not match the page writer's KV heads [%u][%u]", norm_config->num_heads,
                norm_config->head_dim, page_config->num_kv_heads, page_config->head_dim);
    KHM_REQUIRE(norm_config->dtype == KHM_DTYPE_BF16, "the fused K RMSNorm/RoPE page write takes BF16 K and V rows");
    const khm_kv_page_write_buffers page_buffers{buffers->pages, buffers->k, buffers->v, buffers->req_slots, buffers->flat_token_indices,
                                                 buffers->page_ids};
    PageWriteParams pages{};
    if (int status = fill_page_write_params(page_config, shape, &page_buffers, num_active_tokens, page_table_index, replay_parameters, &pages))
        return status;
    RmsNormRopeParams p{};
    if (int status = fill_rms_norm_rope_params(norm_config, shape->num_total_token_writes, buffers->k, buffers->norm_weight,
                                               buffers->flat_token_indices, nullptr, num_active_tokens, replay_parameters, &p))
        return status;
    const RowsGeometry geometry = rows_geometry(*norm_config, shape->num_total_token_writes,
                                                (uintptr_t)p.input | (uintptr_t)pages.flat_v | (uintptr_t)p.norm_weight | (uintptr_t)pages.pages, kPageRowsInFlight);
    if (!geometry.fits || page_config->page_bytes % 16 != 0)
        return fail(KHM_ERR_UNSUPPORTED, "the fused K RMSNorm/RoPE page write needs 16-byte aligned buffers, head_dim <= 512, and head_dim and "
                                         "rope_dim / 2 multiples of 8: run khm_rms_norm_rope and khm_kv_page_write instead");
    p.tokens_per_block = geometry.tokens_per_block;
    p.row_slots_per_token_shift = geometry.slot_shift;
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    const bool weight_bf16 = norm_config->norm_weight_dtype == KHM_DTYPE_BF16, fp8_pages = page_config->kv_dtype == KHM_DTYPE_FP8_E4M3FN;
    auto launch = [&](auto weight_tag, auto fp8_tag) {
        typedef decltype(weight_tag) W;
        constexpr bool FP8 = decltype(fp8_tag)::value;
#define KHM_ROWS_CASE(LPR, PARTNER)                                                                                                    \
    if (geometry.lanes_per_row == LPR && geometry.partner == PARTNER) {                                                                \
        KHM_LAUNCH((k_norm_rope_page_write_kernel<W, LPR, PARTNER, FP8>), geometry.grid, dim3(256), 0, hip_stream, p, pages);   \
        return;                                                                                                                        \
    }
        KHM_ROWS_CASES(KHM_ROWS_CASE)
#undef KHM_ROWS_CASE
    };
    if (weight_bf16 && fp8_pages) launch(uint16_t{}, std::true_type{});
    else if (weight_bf16) launch(uint16_t{}, std::false_type{});
    else if (fp8_pages) launch(float{}, std::true_type{});
    else launch(float{}, std::false_type{});
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "K RMSNorm/RoPE page write launch failed: %s", hipGetErrorString(status));
    return KHM_OK;
}

static bool same_rotation(const khm_rms_norm_rope_config& a, const khm_rms_norm_rope_config& b) {
    const khm_rope_scaling &x = a.rope_scaling, &y = b.rope_scaling;
    return a.head_dim == b.head_dim && a.rope_dim == b.rope_dim && a.rope_theta == b.rope_theta && x.kind == y.kind &&
           (x.kind != KHM_ROPE_SCALING_YARN ||
            (x.factor == y.factor && x.attention_factor == y.attention_factor && x.beta_fast == y.beta_fast && x.beta_slow == y.beta_slow &&
             x.original_max_position_embeddings == y.original_max_position_embeddings && x.truncate == y.truncate));
}

// The projection split, Q RMSNorm + RoPE, K RMSNorm + RoPE and the K/V page write in one launch: what GQA::record enqueues
// between the input projection and the SDPA (crates/inference-executor-metal/src/attn/gqa/backend.rs:358-412), with no
// q, k, v or normalised-K rows in memory in between.  Outputs are exactly what khm_gqa_qgkv_split (or khm_gqa_qkv_split),
// khm_rms_norm_rope on the Q rows and khm_k_norm_rope_page_write leave in q_output, gate_output and the pages.
extern "C" int khm_gqa_projection_norm_rope_page_write(uint32_t gated, const khm_rms_norm_rope_config* q_norm_config,
                                                       const khm_rms_norm_rope_config* k_norm_config,
                                                       const khm_kv_page_write_config* page_config, const khm_kv_page_write_shape* shape,
                                                       const khm_gqa_projection_norm_rope_page_write_buffers* buffers,
                                                       khm_replay_u32 num_active_tokens, khm_replay_u32 page_table_index,
                                                       const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(q_norm_config != nullptr && k_norm_config != nullptr && page_config != nullptr && shape != nullptr && buffers != nullptr,
                "configs, shape and buffers must not be null");
    if (int status = validate_rms_norm_rope_config(q_norm_config)) return status;
    if (int status = validate_rms_norm_rope_config(k_norm_config)) return status;
    KHM_REQUIRE(k_norm_config->num_heads == page_config->num_kv_heads && k_norm_config->head_dim == page_config->head_dim,
                "K RMSNorm/RoPE rows [%u][%u] do not match the page writer's KV heads [%u][%u]", k_norm_config->num_heads,
                k_norm_config->head_dim, page_config->num_kv_heads, page_config->head_dim);
    KHM_REQUIRE(q_norm_config->dtype == KHM_DTYPE_BF16 && k_norm_config->dtype == KHM_DTYPE_BF16,
                "the fused projection RMSNorm/RoPE page write takes BF16 projection rows");
    KHM_REQUIRE(same_rotation(*q_norm_config, *k_norm_config) && q_norm_config->norm_weight_dtype == k_norm_config->norm_weight_dtype,
                "the fused projection RMSNorm/RoPE page write needs the same head_dim, rotation and weight dtype for Q and K");
    const uint32_t tokens = shape->num_total_token_writes;
    const uint32_t head_dim = q_norm_config->head_dim, hq = q_norm_config->num_heads, hkv = k_norm_config->num_heads;
    const uint64_t q_heads_in_row = (gated ? 2ull : 1ull) * hq;
    const uint64_t row_heads = q_heads_in_row + 2ull * hkv;
    const __uint128_t elements = (__uint128_t)tokens * row_heads * head_dim;
    KHM_REQUIRE(tokens > 0 && elements <= 0xffffffffull, "%s elements exceeds the shader u32 count domain",
                gated ? "GQA projection" : "ungated GQA projection");
    const uint64_t width = row_heads * head_dim;
    const uint64_t q_bytes = (uint64_t)tokens * hq * head_dim * 2;
    KHM_REQUIRE(buffers->projection.ptr != nullptr && buffers->projection.len_bytes >= (uint64_t)elements * 2,
                "projection buffer holds %llu bytes, needs %llu", (unsigned long long)buffers->projection.len_bytes,
                (unsigned long long)((uint64_t)elements * 2));
    if (gated)
        KHM_REQUIRE(buffers->gate_output.ptr != nullptr && buffers->gate_output.len_bytes >= q_bytes, "gate_output buffer holds %llu bytes, needs %llu",
                    (unsigned long long)buffers->gate_output.len_bytes, (unsigned long long)q_bytes);
    // K and V rows as windows of the projection rows
    const uint64_t k_offset = q_heads_in_row * head_dim * 2, v_offset = k_offset + (uint64_t)hkv * head_dim * 2;
    uint8_t* base = static_cast<uint8_t*>(buffers->projection.ptr);
    const khm_buffer k_window{base + k_offset, buffers->projection.len_bytes - k_offset};
    const khm_buffer v_window{base + v_offset, buffers->projection.len_bytes - v_offset};
    const khm_kv_page_write_buffers page_buffers{buffers->pages, k_window, v_window, buffers->req_slots, buffers->flat_token_indices, buffers->page_ids};
    PageWriteParams pages{};
    if (int status = fill_page_write_params(page_config, shape, &page_buffers, num_active_tokens, page_table_index, replay_parameters, &pages))
        return status;
    RmsNormRopeParams p{}, k_params{};
    if (int status = fill_rms_norm_rope_params(q_norm_config, tokens, buffers->projection, buffers->q_norm_weight, buffers->flat_token_indices,
                                               &buffers->q_output, num_active_tokens, replay_parameters, &p))
        return status;
    if (int status = fill_rms_norm_rope_params(k_norm_config, tokens, k_window, buffers->k_norm_weight, buffers->flat_token_indices, nullptr,
                                               num_active_tokens, replay_parameters, &k_params))
        return status;
    const uintptr_t address_bits = (uintptr_t)base | (uintptr_t)p.output | (uintptr_t)p.norm_weight | (uintptr_t)k_params.norm_weight |
                                   (uintptr_t)pages.pages | (uintptr_t)buffers->gate_output.ptr | (uintptr_t)(width * 2);
    const RowsGeometry q_geometry = rows_geometry(*q_norm_config, tokens, address_bits);
    const RowsGeometry k_geometry = rows_geometry(*k_norm_config, tokens, address_bits, kPageRowsInFlight);
    if (!q_geometry.fits || !k_geometry.fits || page_config->page_bytes % 16 != 0)
        return fail(KHM_ERR_UNSUPPORTED, "the fused projection RMSNorm/RoPE page write needs 16-byte aligned buffers and rows, head_dim <= 512, and "
                                         "head_dim and rope_dim / 2 multiples of 8: run the split, khm_rms_norm_rope and khm_kv_page_write instead");
    p.tokens_per_block = q_geometry.tokens_per_block;
    p.row_slots_per_token_shift = q_geometry.slot_shift;
    p.input_row_stride = (uint32_t)width;
    p.input_head_stride = gated ? 2 * head_dim : head_dim;
    p.gate_output = gated ? buffers->gate_output.ptr : nullptr;
    const RowsRole k_role{k_params.input, k_params.norm_weight, nullptr, nullptr, hkv, (uint32_t)width, head_dim, (uint32_t)width, k_norm_config->eps,
                          k_geometry.tokens_per_block, k_geometry.slot_shift};
    const uint64_t q_blocks = (uint64_t)q_geometry.grid.x * q_geometry.grid.y, k_blocks = (uint64_t)k_geometry.grid.x * k_geometry.grid.y;
    KHM_REQUIRE(q_blocks + k_blocks <= 0x7fffffffull, "the fused projection RMSNorm/RoPE page write needs %llu blocks, more than one launch covers",
                (unsigned long long)(q_blocks + k_blocks));
    // (Running the blocks in token order instead, the Q blocks of four tokens and then their K block, changes nothing:
    // 212.6 against 213.5 us on 16384 tokens; two or one row group in flight in the Q blocks: 218.5 / 217.1 against 214.2 us.)
    const ProjectionBlocks blocks{(uint32_t)q_blocks, q_geometry.grid.x, k_geometry.grid.x};
    const dim3 grid((uint32_t)(q_blocks + k_blocks));
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    const bool weight_bf16 = q_norm_config->norm_weight_dtype == KHM_DTYPE_BF16, fp8_pages = page_config->kv_dtype == KHM_DTYPE_FP8_E4M3FN;
    auto launch = [&](auto weight_tag, auto fp8_tag, auto gated_tag) {
        typedef decltype(weight_tag) W;
        constexpr bool FP8 = decltype(fp8_tag)::value, GATED = decltype(gated_tag)::value;
#define KHM_ROWS_CASE(LPR, PARTNER)                                                                                                          \
    if (q_geometry.lanes_per_row == LPR && q_geometry.partner == PARTNER) {                                                                  \
        KHM_LAUNCH((projection_norm_rope_page_write_kernel<W, LPR, PARTNER, FP8, GATED>), grid, dim3(256), 0, hip_stream, p, k_role, \
                           pages, blocks);                                                                                                   \
        return;                                                                                                                              \
    }
        KHM_ROWS_CASES(KHM_ROWS_CASE)
#undef KHM_ROWS_CASE
    };
    auto with_gate = [&](auto weight_tag, auto fp8_tag) {
        if (gated) launch(weight_tag, fp8_tag, std::true_type{});
        else launch(weight_tag, fp8_tag, std::false_type{});
    };
    if (weight_bf16 && fp8_pages) with_gate(uint16_t{}, std::true_type{});
    else if (weight_bf16) with_gate(uint16_t{}, std::false_type{});
    else if (fp8_pages) with_gate(float{}, std::true_type{});
    else with_gate(float{}, std::false_type{});
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "projection RMSNorm/RoPE page write launch failed: %s", hipGetErrorString(status));
    return KHM_OK;
}
