// K/V page writer and the device side of the FP8 codec: host validation, kernels and launches.
//
// Mirrors kv_page_write::{Config, Shape, Buffers, Compute, Invocation}
// (crates/inference-backend-metal/src/components/gqa/kv_page_write.rs:60-283) and the kernel
// gqa_kv_page_write_fp8_e4m3fn (.../metal/gqa_kv_page_write.metal:33-110): each token write scatters its bf16 K and V
// rows through the page table into page layout [K|V][Hkv][tokens_per_page][D].  The reference stores FP8 E4M3FN only;
// here the page element type is a parameter, so that the bf16 pages of the benchmark configs are produced by the same
// component.  Nothing here allocates or synchronizes.
#include <hip/hip_runtime.h>

#include "common.h"
#include "device_math.hip.h"
#include "device_params.h"
#include "fp8_device.hip.h"
#include "page_write_params.h"

namespace khm {


// A block serves kWritesPerBlock consecutive token writes; a thread moves eight consecutive dims of one KV head's row for
// each of them, for K and for V: a 16-byte load each, then a 16-byte (bf16 pages) or 8-byte (FP8 pages) streaming store
// each.  The request slots, positions, page ids and rows of all of a block's writes are requested before the first is
// used, so the chain slot/position -> page id -> store is walked for four tokens at once (16384 writes of 8 heads x 128
// dims into FP8 pages: 18.7 us; 20.8 us with one write per block and the walk as scalar work, 20.4 / 22.2 us with eight /
// sixteen writes per block).  Head dims that are no multiple of eight take the scalar tail.
constexpr int kWritesPerBlock = 4;
template <bool FP8_PAGES>
__global__ __launch_bounds__(1024) void kv_page_write_kernel(const PageWriteParams p) {
    const uint32_t num_active = resolve_u32(p.num_active_token_writes, p.replay_parameters);
    const uint32_t first_write = blockIdx.x * kWritesPerBlock;
    if (first_write >= num_active) return;
    const uint32_t chunks_per_row = (p.head_dim + 7) / 8;
    const uint32_t in_write = blockIdx.y * blockDim.x + threadIdx.x;
    if (in_write >= p.num_kv_heads * chunks_per_row) return;
    const uint32_t head = in_write / chunks_per_row;
    const uint32_t dim = (in_write - head * chunks_per_row) * 8;
    const uint32_t layer = resolve_u32(p.layer_index, p.replay_parameters);
    constexpr uint32_t kElementBytes = FP8_PAGES ? 1 : 2;

    bool live[kWritesPerBlock];
    uint32_t write_index[kWritesPerBlock], req_slot[kWritesPerBlock], token[kWritesPerBlock];
#pragma unroll
    for (int w = 0; w < kWritesPerBlock; ++w) {
        live[w] = first_write + w < num_active;
        write_index[w] = live[w] ? first_write + w : first_write;
        req_slot[w] = p.req_slots[write_index[w]];
        token[w] = p.flat_token_indices[write_index[w]];
    }
    if (p.head_dim % 8 == 0) {
        uint4 k[kWritesPerBlock], v[kWritesPerBlock];
        PageTarget target[kWritesPerBlock];
#pragma unroll
        for (int w = 0; w < kWritesPerBlock; ++w) {
            const uint64_t source = ((uint64_t)write_index[w] * p.num_kv_heads + head) * p.head_dim + dim;
            k[w] = *reinterpret_cast<const uint4*>(p.flat_k + source);
            v[w] = *reinterpret_cast<const uint4*>(p.flat_v + source);
            target[w] = page_target_of(p, req_slot[w], token[w], layer, head, dim, kElementBytes);
        }
#pragma unroll
        for (int w = 0; w < kWritesPerBlock; ++w) {
            if (!live[w]) continue;
            uint8_t* k_target = p.pages + target[w].k_offset;
            uint8_t* v_target = k_target + target[w].v_distance;
            if constexpr (FP8_PAGES) {
                store_streaming(k_target, bf16x8_bits_to_fp8x8_e4m3fn(k[w]));
                store_streaming(v_target, bf16x8_bits_to_fp8x8_e4m3fn(v[w]));
            } else {
                store_streaming(k_target, k[w]);
                store_streaming(v_target, v[w]);
            }
        }
        return;
    }
#pragma unroll
    for (int w = 0; w < kWritesPerBlock; ++w) {
        if (!live[w]) continue;
        const PageTarget target = page_target_of(p, req_slot[w], token[w], layer, head, dim, kElementBytes);
        uint8_t* k_target = p.pages + target.k_offset;
        uint8_t* v_target = k_target + target.v_distance;
        const uint64_t source = ((uint64_t)write_index[w] * p.num_kv_heads + head) * p.head_dim + dim;
        for (uint32_t i = 0; i < 8 && dim + i < p.head_dim; ++i) {
            const uint32_t k = p.flat_k[source + i], v = p.flat_v[source + i];
            if constexpr (FP8_PAGES) {
                k_target[i] = (uint8_t)bf16_bits_to_fp8_e4m3fn(k);
                v_target[i] = (uint8_t)bf16_bits_to_fp8_e4m3fn(v);
            } else {
                reinterpret_cast<uint16_t*>(k_target)[i] = (uint16_t)k;
                reinterpret_cast<uint16_t*>(v_target)[i] = (uint16_t)v;
            }
        }
    }
}

// Element-wise codec kernels: what the attention kernels and the page writer do per element, exposed so that the device
// conversions can be checked against the host codec over every code and every bf16 pattern.
__global__ __launch_bounds__(256) void fp8_decode_kernel(const uint8_t* codes, uint16_t* bf16_out, uint64_t count) {
    const uint64_t gid = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (gid >= count) return;
    if (gid + 8 <= count) {
        *reinterpret_cast<uint4*>(bf16_out + gid) = fp8x8_to_bf16x8(*reinterpret_cast<const uint2*>(codes + gid));
        return;
    }
    for (uint64_t i = gid; i < count; ++i) bf16_out[i] = (uint16_t)(fp8x2_to_bf16x2<false>(codes[i]) & 0xffffu);
}

// Thread t encodes elements 8t .. 8t+7 with the eight-wide conversion the page writers use; what is left of the last
// group goes through the paired conversion, and a last odd element through the integer encoder.
__global__ __launch_bounds__(256) void fp8_encode_kernel(const uint16_t* bf16_in, uint8_t* codes, uint64_t count) {
    const uint64_t gid = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (gid >= count) return;
    if (gid + 8 <= count) {
        *reinterpret_cast<uint2*>(codes + gid) = bf16x8_bits_to_fp8x8_e4m3fn(*reinterpret_cast<const uint4*>(bf16_in + gid));
        return;
    }
    uint64_t i = gid;
    for (; i + 1 < count; i += 2) {
        const uint32_t both = bf16x2_bits_to_fp8x2_e4m3fn((uint32_t)bf16_in[i] | ((uint32_t)bf16_in[i + 1] << 16));
        codes[i] = (uint8_t)(both & 0xffu);
        codes[i + 1] = (uint8_t)(both >> 8);
    }
    if (i < count) codes[i] = (uint8_t)bf16_bits_to_fp8_e4m3fn(bf16_in[i]);
}

static DeviceReplayU32 to_device_replay(khm_replay_u32 value) { return DeviceReplayU32{value.is_parameter, value.value}; }

static int check_page_write_launch(const char* what) {
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(status));
    return KHM_OK;
}

}  // namespace khm

using namespace khm;

// kv_page_write::Config::num_tokens_per_page (kv_page_write.rs:76-89), with the page element size made explicit.
extern "C" uint32_t khm_kv_page_write_num_tokens_per_page(const khm_kv_page_write_config* config) {
    if (config == nullptr) return 0;
    const uint64_t bytes_per_token = (uint64_t)config->num_kv_heads * config->head_dim * 2 * kv_element_bytes(config->kv_dtype);
    if (bytes_per_token == 0 || bytes_per_token > 0xffffffffull || config->page_bytes % bytes_per_token != 0) return 0;
    return (uint32_t)(config->page_bytes / bytes_per_token);
}

// see page_write_params.h
int khm::fill_page_write_params(const khm_kv_page_write_config* config, const khm_kv_page_write_shape* shape,
                                const khm_kv_page_write_buffers* buffers, khm_replay_u32 num_active_token_writes,
                                khm_replay_u32 page_table_index, const uint32_t* replay_parameters, PageWriteParams* out) {
    KHM_REQUIRE(config != nullptr && shape != nullptr && buffers != nullptr, "config, shape and buffers must not be null");
    // Config::validate (kv_page_write.rs:67-75)
    KHM_REQUIRE(config->num_kv_heads > 0, "GQA KV page write requires KV heads");
    KHM_REQUIRE(config->head_dim > 0, "GQA KV page write requires a head dimension");
    KHM_REQUIRE(config->dtype == KHM_DTYPE_BF16, "GQA FP8 KV page write requires BF16 source tensors");
    KHM_REQUIRE(config->kv_dtype == KHM_DTYPE_FP8_E4M3FN || config->kv_dtype == KHM_DTYPE_BF16, "GQA K/V pages must be BF16 or FP8 E4M3FN");
    const uint32_t tokens_per_page = khm_kv_page_write_num_tokens_per_page(config);
    KHM_REQUIRE(tokens_per_page > 0, "GQA page_bytes must be divisible by the K/V bytes per token");
    // Shape::validate (kv_page_write.rs:121-128)
    const khm_page_table_layout& layout = shape->page_table_layout;
    KHM_REQUIRE(shape->num_total_token_writes > 0, "GQA KV page write requires token writes");
    KHM_REQUIRE(layout.num_req_slots > 0 && layout.num_blocks > 0 && layout.num_gqa_layers > 0 && layout.num_page_ids_per_block > 0,
                "GQA page table requires request slots, layers, blocks and page ids per block");
    const __uint128_t threads = (__uint128_t)shape->num_total_token_writes * config->num_kv_heads * config->head_dim;
    KHM_REQUIRE(threads <= 0xffffffffull, "GQA KV page-write threads exceeds the shader u32 count domain");
    // Invocation::validate (kv_page_write.rs:264-279)
    if (!num_active_token_writes.is_parameter) {
        KHM_REQUIRE(num_active_token_writes.value >= 1 && num_active_token_writes.value <= shape->num_total_token_writes,
                    "num_active_token_writes=%u is outside its replay domain [1, %u]", num_active_token_writes.value,
                    shape->num_total_token_writes);
    } else {
        KHM_REQUIRE(replay_parameters != nullptr, "num_active_token_writes is a replay parameter but no parameter block was given");
    }
    if (!page_table_index.is_parameter) {
        KHM_REQUIRE(page_table_index.value < layout.num_gqa_layers, "page_table_index=%u is outside its replay domain [0, %u]",
                    page_table_index.value, layout.num_gqa_layers - 1);
    } else {
        KHM_REQUIRE(replay_parameters != nullptr, "page_table_index is a replay parameter but no parameter block was given");
    }
    const uint64_t flat_bytes = (uint64_t)threads * 2;
    const uint64_t index_bytes = (uint64_t)shape->num_total_token_writes * 4;
    const uint64_t table_bytes = (uint64_t)layout.num_req_slots * layout.num_gqa_layers * layout.num_blocks * layout.num_page_ids_per_block * 4;
    KHM_REQUIRE(buffers->pages.ptr != nullptr && buffers->pages.len_bytes >= config->page_bytes, "pages buffer holds %llu bytes, needs %llu",
                (unsigned long long)buffers->pages.len_bytes, (unsigned long long)config->page_bytes);
    KHM_REQUIRE(buffers->flat_k.ptr != nullptr && buffers->flat_k.len_bytes >= flat_bytes, "flat_k buffer holds %llu bytes, needs %llu",
                (unsigned long long)buffers->flat_k.len_bytes, (unsigned long long)flat_bytes);
    KHM_REQUIRE(buffers->flat_v.ptr != nullptr && buffers->flat_v.len_bytes >= flat_bytes, "flat_v buffer holds %llu bytes, needs %llu",
                (unsigned long long)buffers->flat_v.len_bytes, (unsigned long long)flat_bytes);
    KHM_REQUIRE(buffers->req_slots.ptr != nullptr && buffers->req_slots.len_bytes >= index_bytes, "req_slots buffer holds %llu bytes, needs %llu",
                (unsigned long long)buffers->req_slots.len_bytes, (unsigned long long)index_bytes);
    KHM_REQUIRE(buffers->flat_token_indices.ptr != nullptr && buffers->flat_token_indices.len_bytes >= index_bytes,
                "flat_token_indices buffer holds %llu bytes, needs %llu", (unsigned long long)buffers->flat_token_indices.len_bytes,
                (unsigned long long)index_bytes);
    KHM_REQUIRE(buffers->page_ids.ptr != nullptr && buffers->page_ids.len_bytes >= table_bytes, "page_ids buffer holds %llu bytes, needs %llu",
                (unsigned long long)buffers->page_ids.len_bytes, (unsigned long long)table_bytes);

    PageWriteParams p{};
    p.pages = static_cast<uint8_t*>(buffers->pages.ptr);
    p.flat_k = static_cast<const uint16_t*>(buffers->flat_k.ptr);
    p.flat_v = static_cast<const uint16_t*>(buffers->flat_v.ptr);
    p.req_slots = static_cast<const uint32_t*>(buffers->req_slots.ptr);
    p.flat_token_indices = static_cast<const uint32_t*>(buffers->flat_token_indices.ptr);
    p.page_ids = static_cast<const uint32_t*>(buffers->page_ids.ptr);
    p.replay_parameters = replay_parameters;
    p.num_active_token_writes = to_device_replay(num_active_token_writes);
    p.layer_index = to_device_replay(page_table_index);
    p.page_bytes = config->page_bytes;
    p.num_kv_heads = config->num_kv_heads;
    p.head_dim = config->head_dim;
    p.tokens_per_page = tokens_per_page;
    p.num_gqa_layers = layout.num_gqa_layers;
    p.num_blocks = layout.num_blocks;
    p.num_page_ids_per_block = layout.num_page_ids_per_block;
    *out = p;
    return KHM_OK;
}

extern "C" int khm_kv_page_write(const khm_kv_page_write_config* config, const khm_kv_page_write_shape* shape,
                                 const khm_kv_page_write_buffers* buffers, khm_replay_u32 num_active_token_writes,
                                 khm_replay_u32 page_table_index, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    PageWriteParams p{};
    if (int status = fill_page_write_params(config, shape, buffers, num_active_token_writes, page_table_index, replay_parameters, &p)) return status;
    const uint64_t chunks_per_write = (uint64_t)config->num_kv_heads * ((config->head_dim + 7) / 8);
    const uint32_t block_threads = (uint32_t)(chunks_per_write >= 1024 ? 1024 : (chunks_per_write + 63) / 64 * 64);
    const uint64_t chunk_blocks = (chunks_per_write + block_threads - 1) / block_threads;
    KHM_REQUIRE(chunk_blocks <= 65535, "GQA KV page write: %llu chunks per token write exceed the launch grid", (unsigned long long)chunks_per_write);
    const dim3 grid((shape->num_total_token_writes + kWritesPerBlock - 1) / kWritesPerBlock, (uint32_t)chunk_blocks);
    if (config->kv_dtype == KHM_DTYPE_FP8_E4M3FN) {
        KHM_LAUNCH(kv_page_write_kernel<true>, grid, dim3(block_threads), 0, static_cast<hipStream_t>(stream), p);
    } else {
        KHM_LAUNCH(kv_page_write_kernel<false>, grid, dim3(block_threads), 0, static_cast<hipStream_t>(stream), p);
    }
    return check_page_write_launch("KV page write");
}

extern "C" int khm_fp8_e4m3_to_bf16_device(khm_buffer codes, khm_buffer bf16_out, uint64_t count, void* stream) {
    clear_error();
    KHM_REQUIRE(count > 0, "FP8 decode requires elements");
    KHM_REQUIRE(codes.ptr != nullptr && codes.len_bytes >= count, "codes buffer holds %llu bytes, needs %llu",
                (unsigned long long)codes.len_bytes, (unsigned long long)count);
    KHM_REQUIRE(bf16_out.ptr != nullptr && bf16_out.len_bytes >= count * 2, "bf16_out buffer holds %llu bytes, needs %llu",
                (unsigned long long)bf16_out.len_bytes, (unsigned long long)(count * 2));
    KHM_REQUIRE(reinterpret_cast<uintptr_t>(codes.ptr) % 8 == 0 && reinterpret_cast<uintptr_t>(bf16_out.ptr) % 16 == 0,
                "FP8 decode buffers must be 8- and 16-byte aligned");
    const uint64_t threads = (count + 7) / 8;
    KHM_LAUNCH(fp8_decode_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint8_t*>(codes.ptr), static_cast<uint16_t*>(bf16_out.ptr), count);
    return check_page_write_launch("FP8 decode");
}

extern "C" int khm_bf16_to_fp8_e4m3_device(khm_buffer bf16_in, khm_buffer codes, uint64_t count, void* stream) {
    clear_error();
    KHM_REQUIRE(count > 0, "FP8 encode requires elements");
    KHM_REQUIRE(bf16_in.ptr != nullptr && bf16_in.len_bytes >= count * 2, "bf16_in buffer holds %llu bytes, needs %llu",
                (unsigned long long)bf16_in.len_bytes, (unsigned long long)(count * 2));
    KHM_REQUIRE(codes.ptr != nullptr && codes.len_bytes >= count, "codes buffer holds %llu bytes, needs %llu",
                (unsigned long long)codes.len_bytes, (unsigned long long)count);
    KHM_REQUIRE(reinterpret_cast<uintptr_t>(codes.ptr) % 8 == 0 && reinterpret_cast<uintptr_t>(bf16_in.ptr) % 16 == 0,
                "FP8 encode buffers must be 8- and 16-byte aligned");
    const uint64_t threads = (count + 7) / 8;
    KHM_LAUNCH(fp8_encode_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(bf16_in.ptr), static_cast<uint8_t*>(codes.ptr), count);
    return check_page_write_launch("FP8 encode");
}
