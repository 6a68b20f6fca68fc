// Kernel argument blocks shared by the host launchers and the gfx950 kernels.
#pragma once
#include <stdint.h>

namespace khm {

// ReplayU32: a fixed value or an index into the device parameter block.
struct DeviceReplayU32 {
    uint32_t is_parameter;
    uint32_t value;
};

enum MapOutputMode : uint32_t {
    kMapPartialBf16 = 0,  // normalized partial, bf16, plus f32 (sum, natural-log max)
    kMapPartialF32 = 1,   // normalized partial, f32, plus stats
    kMapDirectBf16 = 2,   // final bf16 output, no stats
};

// Arguments of the split-KV Map kernels (decode, verify and the tiled prefill kernel).
struct MapParams {
    const uint16_t* q;                  // bf16 [T][Hq][D]
    const uint8_t* kv_pages;            // [P][page_bytes]
    const uint32_t* req_slots;          // [T]
    const uint32_t* page_ids;           // [R][L][NB][PPB]
    const uint32_t* visible_ranges;     // [T][2] or nullptr (sliced-KV: template range only)
    const uint32_t* q_token_ranges;     // [R][2] or nullptr (sliced-KV: range i = token i)
    const uint32_t* templates;          // [M][3]
    float* exp_sums;                    // [M][Hq][max_q_tokens]
    float* max_logits;                  // [M][Hq][max_q_tokens]
    void* out;                          // partial [M][Hq][max_q_tokens][D] or output [T][Hq][D]
    const uint32_t* replay_parameters;  // device u32 block or nullptr
    DeviceReplayU32 layer_index;
    DeviceReplayU32 num_active_tokens;
    DeviceReplayU32 num_active_q_token_tiles;  // sliced-KV: same as num_active_tokens
    DeviceReplayU32 num_active_kv_splits;
    uint64_t page_bytes;
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t q_heads_per_kv_head;
    uint32_t max_q_heads;                // Q heads per block (<= q_heads_per_kv_head)
    uint32_t num_q_head_ranges;          // ceil(q_heads_per_kv_head / max_q_heads)
    uint32_t max_q_tokens;               // Q tokens per range (1 for sliced-KV)
    uint32_t tokens_per_page;            // 8, 16 or 32
    uint32_t tokens_per_page_shift;
    uint32_t num_gqa_layers;
    uint32_t pages_per_request_layer;    // num_blocks * num_page_ids_per_block
    uint32_t output_mode;                // MapOutputMode
    float scale_log2e;                   // scale * log2(e)
    // Fused Reduce (optional): the last block to finish a (Q range, head group) merges its partials.
    const uint32_t* cu_partial_outputs;  // [R + 1]
    uint32_t* arrival_counters;          // [R][gridDim.y], zero before the first launch; the merging block re-arms its counter
    uint16_t* final_output;              // bf16 [T][Hq][D]
    const uint16_t* gates;               // bf16 [T][Hq][D] or nullptr: gate of the fused Reduce, or of direct output
};

// Arguments of the flat (sliced-KV) and ranged (sliced-Q) Reduce kernels.
struct ReduceParams {
    const float* exp_sums;
    const float* max_logits;
    const void* partial;
    const uint32_t* q_token_ranges;      // sliced-Q only
    const uint32_t* cu_partial_outputs;
    const uint16_t* gates;               // bf16 [T][Hq][D] or nullptr
    uint16_t* output;                    // bf16 [T][Hq][D]
    const uint32_t* replay_parameters;
    DeviceReplayU32 num_active;          // tokens (sliced-KV) or Q-token tiles (sliced-Q)
    uint32_t num_q_heads;
    uint32_t head_dim;
    uint32_t max_q_tokens;
    uint32_t partial_is_f32;
};

struct GateParams {
    const void* attention;
    const void* gates;
    void* output;
    const uint32_t* replay_parameters;
    DeviceReplayU32 num_active_tokens;
    uint32_t values_per_token;
    uint32_t is_f32;
};

}  // namespace khm
