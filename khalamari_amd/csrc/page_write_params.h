// Arguments of the K/V page writer, shared by the plain writer and the fused K RMSNorm + RoPE + page write.
#pragma once
#include <stdint.h>

#include "device_params.h"
#include "../../include/khm_gqa_sdpa.h"

namespace khm {

struct PageWriteParams {
    uint8_t* pages;
    const uint16_t* flat_k;             // bf16 [W][Hkv][D]
    const uint16_t* flat_v;
    const uint32_t* req_slots;          // [W]
    const uint32_t* flat_token_indices; // [W]
    const uint32_t* page_ids;           // [R][L][NB][PPB]
    const uint32_t* replay_parameters;
    DeviceReplayU32 num_active_token_writes;
    DeviceReplayU32 layer_index;
    uint64_t page_bytes;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint32_t tokens_per_page;
    uint32_t num_gqa_layers;
    uint32_t num_blocks;
    uint32_t num_page_ids_per_block;
};

// Config::validate, Shape::validate and Invocation::validate of the page writer (kv_page_write.rs:67-75,121-128,264-279)
// plus the buffer-size checks; fills `out` for the launch.  Returns a status code and sets the last error.
int fill_page_write_params(const khm_kv_page_write_config* config, const khm_kv_page_write_shape* shape,
                           const khm_kv_page_write_buffers* buffers, khm_replay_u32 num_active_token_writes,
                           khm_replay_u32 page_table_index, const uint32_t* replay_parameters, PageWriteParams* out);

// Byte offset inside `pages` of element `dim` of KV head `head` in the K plane for one token write, and the distance to
// the same element of the V plane (both in elements of the page type times element_bytes).
struct PageTarget {
    uint64_t k_offset;   // bytes
    uint64_t v_distance; // bytes
};
__device__ __forceinline__ PageTarget page_target_of(const PageWriteParams& p, uint32_t req_slot, uint32_t token, uint32_t layer, uint32_t head,
                                                    uint32_t dim, uint32_t element_bytes) {
    const uint32_t block = token / (p.tokens_per_page * p.num_page_ids_per_block);
    const uint32_t page_index = (token / p.tokens_per_page) % p.num_page_ids_per_block;
    const uint64_t table_index = (((uint64_t)req_slot * p.num_gqa_layers + layer) * p.num_blocks + block) * p.num_page_ids_per_block + page_index;
    const uint64_t page_id = p.page_ids[table_index];
    const uint32_t page_token = token % p.tokens_per_page;
    const uint64_t values_per_plane = (uint64_t)p.num_kv_heads * p.tokens_per_page * p.head_dim;
    const uint64_t in_plane = ((uint64_t)head * p.tokens_per_page + page_token) * p.head_dim + dim;
    return PageTarget{page_id * p.page_bytes + in_plane * element_bytes, values_per_plane * element_bytes};
}

}  // namespace khm
