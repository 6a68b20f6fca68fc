// Host side of the sliced-KV and sliced-Q SDPA components and the sigmoid gate: validation, kernel
// selection and launches.  Mirrors sliced_kv::{Config, Shape, Compute, MapInvocation, ReduceInvocation}
// (crates/inference-backend-metal/src/components/gqa/sdpa/sliced_kv.rs:91-388,548-663),
// sliced_q::{Config, Shape, Compute, ...} (.../sdpa/sliced_q.rs) and activation_gate::Compute
// (.../gqa/activation_gate.rs:35-168).  Nothing here allocates or synchronizes.
#include <hip/hip_runtime.h>

#include <atomic>

#include "common.h"
#include "device_params.h"
#include "reduce_gate.hip.h"
#include "split_kv_map.hip.h"
#include "tile_map.hip.h"

namespace khm {

constexpr int kMapWaves = 4;


typedef void (*MapKernel)(const MapParams);
typedef void (*ReduceKernel)(const ReduceParams);

// Split-KV kernel (waves share nothing); K/V pages bf16 or FP8 E4M3FN.  Every variant that reaches it has one 16-column
// tile: sliced-KV variants carry at most 8 Q heads and sliced-Q variants come here with at most 16 coordinates.
template <bool KV8>
static MapKernel small_tile_kernel_of(uint32_t head_dim, uint32_t column_tiles) {
    if (column_tiles != 1) return nullptr;
    if (head_dim == 128) return split_kv_map_kernel<128, 1, kMapWaves, KV8>;
    if (head_dim == 256) return split_kv_map_kernel<256, 1, kMapWaves, KV8>;
    return nullptr;
}

static MapKernel select_small_tile_kernel(uint32_t head_dim, uint32_t column_tiles, uint32_t kv_dtype) {
    return kv_dtype == KHM_DTYPE_FP8_E4M3FN ? small_tile_kernel_of<true>(head_dim, column_tiles)
                                            : small_tile_kernel_of<false>(head_dim, column_tiles);
}

struct TileKernelChoice {
    MapKernel kernel;
    uint32_t threads;
    uint32_t smem_bytes;
};

// Tiled (LDS-shared K/V) kernel for Q tiles of 17..256 coordinates: speculative-verify blocks (one 16-column tile per
// wave, bandwidth-bound) up to prefill tiles (32 columns per wave, MFMA-bound).
static TileKernelChoice select_tile_kernel(uint32_t head_dim, uint32_t coordinates, uint32_t kv_dtype, bool direct) {
    // The MFMA-bound tiles have a build of their own for computes that only ever write final output: its interior slices
    // do not follow the largest score.  (One kernel holding both kinds of interior loop spills.)  These are the two-
    // column-tile kernels at D 128 and the eight-wave tile at D 256 (523 -> 638 TFLOP/s on 2048-token chunks at
    // Hq24/Hkv4); the bandwidth-bound verify tiles have nothing to gain.
    // Twelve waves of one column tile each for 129..192 coordinates at D 256 (32 tokens x 6 Q heads of a KV head: no idle
    // column, three waves per SIMD), on bf16 and on FP8 pages.
    if (head_dim == 256 && coordinates > 128 && coordinates <= 192) {
        if (kv_dtype == KHM_DTYPE_FP8_E4M3FN) {
            if (direct) return {tile_map_kernel<256, 1, 12, 32, 4, 1, true, true>, 768, (uint32_t)TileSmem<256, 32, 4>::kBytes};
            return {tile_map_kernel<256, 1, 12, 32, 4, 1, true>, 768, (uint32_t)TileSmem<256, 32, 4>::kBytes};
        }
        if (direct) return {tile_map_kernel<256, 1, 12, 32, 4, 1, false, true>, 768, (uint32_t)TileSmem<256, 32, 4, 512, true>::kBytes};
        return {tile_map_kernel<256, 1, 12, 32, 4, 1>, 768, (uint32_t)TileSmem<256, 32, 4, 512, true>::kBytes};
    }
    if (direct && head_dim == 256 && coordinates > 64 && coordinates <= 128) {
        if (kv_dtype == KHM_DTYPE_FP8_E4M3FN)
            return {tile_map_kernel<256, 1, 8, 32, 4, 1, true, true>, 512, (uint32_t)TileSmem<256, 32, 4>::kBytes};
        return {tile_map_kernel<256, 1, 8, 32, 4, 1, false, true>, 512, (uint32_t)TileSmem<256, 32, 4, 512, true>::kBytes};
    }
    if (direct && head_dim == 128 && coordinates > 64) {
        const bool wide = coordinates > 128;
        if (kv_dtype == KHM_DTYPE_FP8_E4M3FN) {
            if (wide) return {tile_map_kernel<128, 2, 8, 64, 4, 1, true, true>, 512, (uint32_t)TileSmem<128, 64, 4>::kBytes};
            return {tile_map_kernel<128, 2, 4, 64, 4, 2, true, true>, 256, (uint32_t)TileSmem<128, 64, 4>::kBytes};
        }
        if (wide) return {tile_map_kernel<128, 2, 8, 64, 4, 1, false, true>, 512, (uint32_t)TileSmem<128, 64, 4, 256, true>::kBytes};
        return {tile_map_kernel<128, 1, 8, 32, 4, 2, false, true>, 512, (uint32_t)TileSmem<128, 32, 4, 256, true>::kBytes};
    }
    if (kv_dtype == KHM_DTYPE_FP8_E4M3FN) {
        if (head_dim == 128) {
            // verify tiles keep the raw codes in LDS (32 KB per block) and decode at the consumer: BK 64 and a fifth stage
            // were measured slower (170 / 167 us against 165 us on a batch of 16 speculative blocks)
            if (coordinates <= 64) return {tile_map_kernel<128, 1, 4, 32, 4, 2, true>, 256, (uint32_t)TileSmem<128, 32, 4, 128>::kBytes};   // raw codes in LDS
            if (coordinates <= 128) return {tile_map_kernel<128, 2, 4, 64, 4, 2, true>, 256, (uint32_t)TileSmem<128, 64, 4>::kBytes};
            return {tile_map_kernel<128, 2, 8, 64, 4, 1, true>, 512, (uint32_t)TileSmem<128, 64, 4>::kBytes};
        }
        if (head_dim == 256) {
            if (coordinates <= 64) return {tile_map_kernel<256, 1, 4, 32, 4, 1, true>, 256, (uint32_t)TileSmem<256, 32, 4, 256>::kBytes};   // raw codes in LDS
            if (coordinates <= 128) return {tile_map_kernel<256, 1, 8, 32, 4, 1, true>, 512, (uint32_t)TileSmem<256, 32, 4>::kBytes};
            return {tile_map_kernel<256, 2, 8, 32, 4, 1, true>, 512, (uint32_t)TileSmem<256, 32, 4>::kBytes};
        }
        return {nullptr, 0, 0};
    }
    if (head_dim == 128) {
        if (coordinates <= 64)
            return {tile_map_kernel<128, 1, 4, 32, 4, 2>, 256, (uint32_t)TileSmem<128, 32, 4, 256, true>::kBytes};  // 64 KB: two blocks per CU
        // 65..128 coordinates on bf16 pages: eight waves of one column tile each, BK 32, 64 KB of LDS, two blocks per CU =
        // four waves per SIMD at 118 VGPRs.  A batch of 2048-token chunks held to 128 columns: 5.13 ms, against 6.93 ms
        // on four waves of two column tiles with BK 64 (and 5.77 ms on eight waves with BK 64 at one block per CU).  FP8
        // pages keep the four-wave tile: a 32-token FP8 tile has fewer load units than eight waves.
        if (coordinates <= 128) return {tile_map_kernel<128, 1, 8, 32, 4, 2>, 512, (uint32_t)TileSmem<128, 32, 4, 256, true>::kBytes};
        return {tile_map_kernel<128, 2, 8, 64, 4, 1>, 512, (uint32_t)TileSmem<128, 64, 4, 256, true>::kBytes};
    }
    if (head_dim == 256) {
        // 65..128 coordinates: eight waves of one column tile each (167 VGPRs, two waves per SIMD) rather than four waves
        // of two (256 VGPRs + 167 AGPRs, one wave per SIMD, nothing to overlap its waits with): 414 -> 527 TFLOP/s on a
        // batch of 2048-token chunks at Hq24/Hkv4.
        if (coordinates <= 64) return {tile_map_kernel<256, 1, 4, 32, 4, 1>, 256, (uint32_t)TileSmem<256, 32, 4, 512, true>::kBytes};
        if (coordinates <= 128) return {tile_map_kernel<256, 1, 8, 32, 4, 1>, 512, (uint32_t)TileSmem<256, 32, 4, 512, true>::kBytes};
        return {tile_map_kernel<256, 2, 8, 32, 4, 1>, 512, (uint32_t)TileSmem<256, 32, 4, 512, true>::kBytes};
    }
    return {nullptr, 0, 0};
}

static ReduceKernel select_reduce_kernel(uint32_t head_dim, bool ranged) {
    if (head_dim == 128) return ranged ? split_kv_reduce_kernel<128, true> : split_kv_reduce_kernel<128, false>;
    if (head_dim == 256) return ranged ? split_kv_reduce_kernel<256, true> : split_kv_reduce_kernel<256, false>;
    return nullptr;
}

// Rows with few partials merge faster one row per thread group (no LDS pass); the shape's average decides.
constexpr uint32_t kFewPartialsPerRow = 16;

static ReduceKernel select_reduce_rows_kernel(uint32_t head_dim, bool ranged) {
    if (head_dim == 128) return ranged ? split_kv_reduce_rows_kernel<128, true> : split_kv_reduce_rows_kernel<128, false>;
    if (head_dim == 256) return ranged ? split_kv_reduce_rows_kernel<256, true> : split_kv_reduce_rows_kernel<256, false>;
    return nullptr;
}

// Launches the Reduce over `units` tokens (flat) or Q ranges (ranged) of `max_q_tokens` token slots each.
static void launch_reduce_kernel(const khm_gqa_sdpa_config& config, const khm_gqa_sdpa_shape& shape, bool ranged, uint32_t units,
                                 uint32_t max_q_tokens, ReduceKernel sliced, const ReduceParams& p, hipStream_t stream) {
    const bool few = (uint64_t)shape.num_total_sdpa_map_task_templates <= (uint64_t)kFewPartialsPerRow * units;
    if (few) {
        const uint64_t rows = (uint64_t)units * max_q_tokens * config.num_q_heads;
        const uint32_t rows_per_block = kReduceThreads / (config.head_dim / 4);
        KHM_LAUNCH(select_reduce_rows_kernel(config.head_dim, ranged), dim3((uint32_t)((rows + rows_per_block - 1) / rows_per_block)),
                           dim3(kReduceThreads), 0, stream, p);
    } else {
        KHM_LAUNCH(sliced, dim3(units * max_q_tokens, config.num_q_heads, 1), dim3(kReduceThreads), 0, stream, p);
    }
}

static DeviceReplayU32 to_device(khm_replay_u32 value) { return DeviceReplayU32{value.is_parameter, value.value}; }

// ReplayU32::validate_range for Fixed values; Parameters are range-checked by whoever fills the block
// (the reference validates them at submit: metal/stream/parameter.rs:186-204).
static int validate_replay(khm_replay_u32 value, uint32_t min_value, uint32_t max_value, const uint32_t* block, const char* name) {
    if (value.is_parameter) {
        KHM_REQUIRE(block != nullptr, "%s is a replay parameter but no parameter block was given", name);
        return KHM_OK;
    }
    KHM_REQUIRE(value.value >= min_value && value.value <= max_value, "%s=%u is outside its replay domain [%u, %u]", name,
                value.value, min_value, max_value);
    return KHM_OK;
}

static int validate_layout(const khm_page_table_layout& layout) {
    KHM_REQUIRE(layout.num_req_slots > 0, "GQA page table requires request slots");
    KHM_REQUIRE(layout.num_blocks > 0, "GQA page table requires blocks");
    KHM_REQUIRE(layout.num_gqa_layers > 0, "GQA page table requires layers");
    KHM_REQUIRE(layout.num_page_ids_per_block > 0, "GQA page table requires page ids per block");
    return KHM_OK;
}

static uint32_t tokens_per_page_of(const khm_gqa_sdpa_config& config) {
    const uint64_t bytes_per_token = (uint64_t)config.num_kv_heads * config.head_dim * 2 * kv_element_bytes(config.kv_dtype);
    if (bytes_per_token == 0 || bytes_per_token > 0xffffffffull || config.page_bytes % bytes_per_token != 0) return 0;
    return (uint32_t)(config.page_bytes / bytes_per_token);
}

// sliced_kv::Config::validate (sliced_kv.rs:101-111) / sliced_q::Config::validate (sliced_q.rs:181-196).
static int validate_component_config(const khm_gqa_sdpa_config* config, bool sliced_q) {
    KHM_REQUIRE(config != nullptr, "GQA SDPA config must not be null");
    KHM_REQUIRE(config->num_q_heads > 0, "GQA SDPA requires Q heads");
    KHM_REQUIRE(config->num_kv_heads > 0, "GQA SDPA requires KV heads");
    KHM_REQUIRE(config->head_dim > 0, "GQA SDPA requires a head dimension");
    KHM_REQUIRE(config->scale > 0.0f, "GQA SDPA scale must be positive");
    KHM_REQUIRE(config->num_q_heads % config->num_kv_heads == 0, "GQA Q heads must be a multiple of KV heads");
    KHM_REQUIRE(config->kv_dtype == KHM_DTYPE_BF16 || config->kv_dtype == KHM_DTYPE_FP8_E4M3FN,
                "GQA K/V pages must be BF16 or FP8 E4M3FN");
    KHM_REQUIRE(config->partial_dtype == KHM_DTYPE_BF16 || config->partial_dtype == KHM_DTYPE_F32,
                "GQA partial outputs must be BF16 or F32");
    const uint32_t tpp = tokens_per_page_of(*config);
    KHM_REQUIRE(tpp > 0, "GQA page_bytes must be divisible by the K/V bytes per token");
    if (int status = validate_layout(config->page_table_layout)) return status;
    if (sliced_q) {
        const bool profile = (config->head_dim == 128 && (tpp == 8 || tpp == 16)) ||
                             (config->head_dim == 256 && (tpp == 8 || tpp == 16 || tpp == 32));
        KHM_REQUIRE(profile,
                    "GQA SplitKV SlicedQ supports only (head_dim, tokens_per_page) profiles (128, 8), (128, 16), (256, 8), "
                    "(256, 16), and (256, 32), got (%u, %u)",
                    config->head_dim, tpp);
        KHM_REQUIRE(config->dtype == KHM_DTYPE_BF16, "GQA SplitKV SlicedQ specializes bf16");
    } else {
        KHM_REQUIRE(config->dtype == KHM_DTYPE_F32 || config->dtype == KHM_DTYPE_BF16, "GQA SDPA dtype must be Float32 or Bfloat16");
    }
    return KHM_OK;
}

static khm_sdpa_config static_config(const khm_gqa_sdpa_config& config) {
    return khm_sdpa_config{config.dtype, config.num_q_heads, config.num_kv_heads, config.head_dim, tokens_per_page_of(config)};
}

static bool mul_overflows_u32(uint64_t a, uint64_t b, uint64_t c = 1) {
    const __uint128_t product = (__uint128_t)a * b * c;
    return product > 0xffffffffull;
}

struct ComputeBase {
    khm_gqa_sdpa_config config;
    khm_sdpa_variant variant;
    khm_gqa_sdpa_shape shape;
    MapKernel map;
    ReduceKernel reduce;
    uint32_t tokens_per_page;
    uint32_t num_q_head_ranges;
    uint32_t map_threads;
    uint32_t map_smem_bytes;
    bool direct;
    bool map_merges_in_kernel;  // the Map kernel can merge a row's partial states itself when its last block arrives
};

static void fill_map_geometry(const ComputeBase& c, MapParams* p) {
    const khm_gqa_sdpa_config& config = c.config;
    p->page_bytes = config.page_bytes;
    p->num_q_heads = config.num_q_heads;
    p->num_kv_heads = config.num_kv_heads;
    p->q_heads_per_kv_head = config.num_q_heads / config.num_kv_heads;
    p->max_q_heads = c.variant.map_max_q_heads;
    p->num_q_head_ranges = c.num_q_head_ranges;
    p->max_q_tokens = c.variant.map_max_q_tokens;
    p->tokens_per_page = c.tokens_per_page;
    p->tokens_per_page_shift = ilog2_u64(c.tokens_per_page);
    p->num_gqa_layers = config.page_table_layout.num_gqa_layers;
    p->pages_per_request_layer = config.page_table_layout.num_blocks * config.page_table_layout.num_page_ids_per_block;
    p->scale_log2e = config.scale * 1.4426950408889634f;
}

static int check_launch(const char* what) {
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(status));
    return KHM_OK;
}

#define KHM_BUFFER_AT_LEAST(buffer, bytes, name)                                                                       \
    KHM_REQUIRE((buffer).ptr != nullptr && (buffer).len_bytes >= (uint64_t)(bytes), "%s buffer holds %llu bytes, needs %llu", \
                name, (unsigned long long)(buffer).len_bytes, (unsigned long long)(bytes))

static uint64_t partial_item_size(const khm_gqa_sdpa_config& config) { return config.partial_dtype == KHM_DTYPE_F32 ? 4 : 2; }

}  // namespace khm

using namespace khm;

struct khm_sliced_kv : ComputeBase {};
struct khm_sliced_q : ComputeBase {};

// ------------------------------------------------------------------------------------------ sizes

extern "C" uint32_t khm_gqa_sdpa_num_tokens_per_page(const khm_gqa_sdpa_config* config) {
    return config ? tokens_per_page_of(*config) : 0;
}

extern "C" uint64_t khm_gqa_sdpa_q_bytes(const khm_gqa_sdpa_config* config, const khm_gqa_sdpa_shape* shape) {
    return (uint64_t)shape->num_total_tokens * config->num_q_heads * config->head_dim * dtype_item_size(config->dtype);
}

extern "C" uint64_t khm_gqa_sdpa_page_ids_bytes(const khm_gqa_sdpa_config* config) {
    const khm_page_table_layout& l = config->page_table_layout;
    return (uint64_t)l.num_req_slots * l.num_gqa_layers * l.num_blocks * l.num_page_ids_per_block * 4;
}

extern "C" uint64_t khm_sliced_kv_partial_output_stats_bytes(const khm_gqa_sdpa_config* config, const khm_gqa_sdpa_shape* shape) {
    return (uint64_t)shape->num_total_sdpa_map_task_templates * config->num_q_heads * 4;
}

extern "C" uint64_t khm_sliced_kv_partial_output_bytes(const khm_gqa_sdpa_config* config, const khm_gqa_sdpa_shape* shape) {
    return (uint64_t)shape->num_total_sdpa_map_task_templates * config->num_q_heads * config->head_dim * partial_item_size(*config);
}

extern "C" uint64_t khm_sliced_q_partial_output_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                                      const khm_gqa_sdpa_shape* shape) {
    return (uint64_t)shape->num_total_sdpa_map_task_templates * config->num_q_heads * variant->map_max_q_tokens *
           config->head_dim * partial_item_size(*config);
}

extern "C" uint64_t khm_sliced_q_partial_output_stats_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                                            const khm_gqa_sdpa_shape* shape) {
    return (uint64_t)shape->num_total_sdpa_map_task_templates * config->num_q_heads * variant->map_max_q_tokens * 4;
}

// ------------------------------------------------------------------------------------------ sliced-KV

static int static_scratch_pointer(unsigned char** out);

extern "C" int khm_sliced_kv_create(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                    const khm_gqa_sdpa_shape* shape, khm_sliced_kv** out) {
    clear_error();
    if (int status = validate_component_config(config, false)) return status;
    KHM_REQUIRE(variant != nullptr && shape != nullptr && out != nullptr, "variant, shape and out must not be null");
    const khm_sdpa_config sdpa = static_config(*config);
    KHM_REQUIRE(variant_supports(*variant, sdpa), "GQA SDPA execution variant does not support the config");
    KHM_REQUIRE(variant->map_kind == KHM_MAP_SLICED_KV, "GQA SplitKV SlicedKv requires a SlicedKv execution variant");
    // Shape::validate (sliced_kv.rs:221-234)
    KHM_REQUIRE(shape->num_total_tokens > 0, "GQA SDPA shape requires tokens");
    KHM_REQUIRE(shape->num_total_sdpa_map_task_templates > 0, "GQA SDPA shape requires Map task templates");
    KHM_REQUIRE(!mul_overflows_u32(shape->num_total_tokens, config->num_q_heads, config->head_dim),
                "GQA SDPA query/output exceeds the shader u32 count domain");
    std::string why;
    if (kernel_family(sdpa, *variant, config->kv_dtype, &why) != 1) return fail(KHM_ERR_UNSUPPORTED, "%s", why.c_str());
    auto* compute = new khm_sliced_kv();
    compute->config = *config;
    compute->variant = *variant;
    compute->shape = *shape;
    compute->tokens_per_page = sdpa.tokens_per_page;
    compute->num_q_head_ranges = div_ceil_u32(sdpa.num_q_heads / sdpa.num_kv_heads, variant->map_max_q_heads);
    compute->direct = false;
    compute->map = select_small_tile_kernel(config->head_dim, div_ceil_u32(variant->map_max_q_heads, 16), config->kv_dtype);
    compute->map_threads = kMapWaves * 64;
    compute->map_smem_bytes = 0;
    compute->map_merges_in_kernel = true;
    compute->reduce = select_reduce_kernel(config->head_dim, false);
    if (compute->map == nullptr || compute->reduce == nullptr) {
        delete compute;
        return fail(KHM_ERR_UNSUPPORTED, "no gfx950 sliced-KV kernel for head_dim %u", config->head_dim);
    }
    // Set-up is the place to look up this device's copy of the static scratch array (khm_sliced_kv_map_reduce_static),
    // so that the entry point itself makes no runtime query on its first call.  Failing here is not an error of create.
    unsigned char* static_scratch = nullptr;
    if (static_scratch_pointer(&static_scratch) != KHM_OK) {
        clear_error();
        (void)hipGetLastError();   // the failed query must not show up as the next launch's error
    }
    *out = compute;
    return KHM_OK;
}

extern "C" void khm_sliced_kv_destroy(khm_sliced_kv* compute) { delete compute; }
extern "C" const void* khm_sliced_kv_map_kernel_id(const khm_sliced_kv* compute) { return reinterpret_cast<const void*>(compute->map); }
extern "C" const void* khm_sliced_kv_reduce_kernel_id(const khm_sliced_kv* compute) {
    return reinterpret_cast<const void*>(compute->reduce);
}

struct FusedReduceArgs {
    const uint32_t* cu_partial_outputs;
    uint32_t* arrival_counters;
    uint16_t* final_output;
    const uint16_t* gates;
};

static int launch_sliced_kv_map(const khm_sliced_kv* compute, const khm_sliced_kv_map_buffers* buffers,
                                khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream,
                                const FusedReduceArgs* fused) {
    KHM_REQUIRE(compute != nullptr && buffers != nullptr, "compute and buffers must not be null");
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    // MapInvocation::validate (sliced_kv.rs:594-613)
    if (int s = validate_replay(page_table_index, 0, config.page_table_layout.num_gqa_layers - 1, replay_parameters, "page_table_index")) return s;
    if (int s = validate_replay(num_active_tokens, 1, shape.num_total_tokens, replay_parameters, "num_active_tokens")) return s;
    if (int s = validate_replay(num_active_kv_splits, 0, shape.num_total_sdpa_map_task_templates, replay_parameters, "num_active_kv_splits")) return s;
    KHM_BUFFER_AT_LEAST(buffers->q, khm_gqa_sdpa_q_bytes(&config, &shape), "q");
    KHM_BUFFER_AT_LEAST(buffers->kv_pages, config.page_bytes, "kv_pages");
    KHM_BUFFER_AT_LEAST(buffers->req_slots, (uint64_t)shape.num_total_tokens * 4, "req_slots");
    KHM_BUFFER_AT_LEAST(buffers->page_ids, khm_gqa_sdpa_page_ids_bytes(&config), "page_ids");
    KHM_BUFFER_AT_LEAST(buffers->sdpa_map_task_templates, (uint64_t)shape.num_total_sdpa_map_task_templates * 12, "sdpa_map_task_templates");
    KHM_BUFFER_AT_LEAST(buffers->partial_exp_sums, khm_sliced_kv_partial_output_stats_bytes(&config, &shape), "partial_exp_sums");
    KHM_BUFFER_AT_LEAST(buffers->partial_max_logits, khm_sliced_kv_partial_output_stats_bytes(&config, &shape), "partial_max_logits");
    KHM_BUFFER_AT_LEAST(buffers->partial_output, khm_sliced_kv_partial_output_bytes(&config, &shape), "partial_output");

    MapParams p{};
    p.q = static_cast<const uint16_t*>(buffers->q.ptr);
    p.kv_pages = static_cast<const uint8_t*>(buffers->kv_pages.ptr);
    p.req_slots = static_cast<const uint32_t*>(buffers->req_slots.ptr);
    p.page_ids = static_cast<const uint32_t*>(buffers->page_ids.ptr);
    p.visible_ranges = nullptr;
    p.q_token_ranges = nullptr;
    p.templates = static_cast<const uint32_t*>(buffers->sdpa_map_task_templates.ptr);
    p.exp_sums = static_cast<float*>(buffers->partial_exp_sums.ptr);
    p.max_logits = static_cast<float*>(buffers->partial_max_logits.ptr);
    p.out = buffers->partial_output.ptr;
    p.replay_parameters = replay_parameters;
    p.layer_index = to_device(page_table_index);
    p.num_active_tokens = to_device(num_active_tokens);
    p.num_active_q_token_tiles = to_device(num_active_tokens);
    p.num_active_kv_splits = to_device(num_active_kv_splits);
    fill_map_geometry(*compute, &p);
    p.output_mode = config.partial_dtype == KHM_DTYPE_F32 ? kMapPartialF32 : kMapPartialBf16;
    if (fused != nullptr) {
        p.cu_partial_outputs = fused->cu_partial_outputs;
        p.arrival_counters = fused->arrival_counters;
        p.final_output = fused->final_output;
        p.gates = fused->gates;
    }
    const dim3 grid(shape.num_total_sdpa_map_task_templates, config.num_kv_heads * compute->num_q_head_ranges, 1);
    KHM_LAUNCH(compute->map, grid, dim3(kMapWaves * 64), 0, static_cast<hipStream_t>(stream), p);
    return check_launch("sliced-KV map");
}

extern "C" int khm_sliced_kv_map(const khm_sliced_kv* compute, const khm_sliced_kv_map_buffers* buffers,
                                 khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                 khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    return launch_sliced_kv_map(compute, buffers, page_table_index, num_active_tokens, num_active_kv_splits, replay_parameters, stream,
                                nullptr);
}

extern "C" uint64_t khm_sliced_kv_arrival_counters_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                                         const khm_gqa_sdpa_shape* shape) {
    const uint32_t ranges = div_ceil_u32(config->num_q_heads / config->num_kv_heads, variant->map_max_q_heads);
    return (uint64_t)shape->num_total_tokens * config->num_kv_heads * ranges * 4;
}

extern "C" int khm_sliced_kv_map_reduce(const khm_sliced_kv* compute, const khm_sliced_kv_map_buffers* map_buffers,
                                        const khm_sliced_kv_reduce_buffers* reduce_buffers, khm_buffer gates, khm_buffer arrival_counters,
                                        khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                        khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(compute != nullptr && map_buffers != nullptr && reduce_buffers != nullptr, "compute and buffers must not be null");
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    KHM_REQUIRE(reduce_buffers->partial_output.ptr == map_buffers->partial_output.ptr &&
                    reduce_buffers->partial_exp_sums.ptr == map_buffers->partial_exp_sums.ptr &&
                    reduce_buffers->partial_max_logits.ptr == map_buffers->partial_max_logits.ptr,
                "fused Map/Reduce needs the same partial buffers on both sides");
    KHM_BUFFER_AT_LEAST(reduce_buffers->cu_sdpa_partial_outputs, ((uint64_t)shape.num_total_tokens + 1) * 4, "cu_sdpa_partial_outputs");
    KHM_BUFFER_AT_LEAST(reduce_buffers->output, khm_gqa_sdpa_q_bytes(&config, &shape), "output");
    KHM_BUFFER_AT_LEAST(arrival_counters, khm_sliced_kv_arrival_counters_bytes(&config, &compute->variant, &shape), "arrival_counters");
    if (gates.ptr != nullptr) KHM_BUFFER_AT_LEAST(gates, khm_gqa_sdpa_q_bytes(&config, &shape), "gates");
    const FusedReduceArgs fused{static_cast<const uint32_t*>(reduce_buffers->cu_sdpa_partial_outputs.ptr),
                                static_cast<uint32_t*>(arrival_counters.ptr), static_cast<uint16_t*>(reduce_buffers->output.ptr),
                                static_cast<const uint16_t*>(gates.ptr)};
    return launch_sliced_kv_map(compute, map_buffers, page_table_index, num_active_tokens, num_active_kv_splits, replay_parameters,
                                stream, &fused);
}

// ---- the fused Map + Reduce without any caller-provided or allocated workspace ----------------------------------------
// For callers that cannot allocate (HIP graph capture, tight serving loops): the partial states and the arrival
// counters of khm_sliced_kv_map_reduce live in a file-scope device array instead of caller buffers.  Each GPU holds its own
// copy of the array at its own address; the address is looked up once per device and only that pointer is ever handed
// to kernels (the array's name is a host-side stand-in, not a device address).
constexpr uint64_t kStaticScratchBytes = 16ull << 20;
constexpr uint64_t kStaticCounterBytes = 256ull << 10;   // arrival counters: a fixed region at the start, never used for anything else
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
// filled when a compute is created on a device (else on the entry point's first call there); concurrent fills store the same value
static std::atomic<unsigned char*> static_scratch_of_device[kMaxDevices];

__global__ __launch_bounds__(256) void clear_u32_kernel(uint32_t* words, uint32_t count) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x;
    if (index < count) words[index] = 0u;
}

static int static_scratch_pointer(unsigned char** out) {
    int device = -1;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "hipGetDevice failed: %s", hipGetErrorString(status));
    KHM_REQUIRE(device >= 0 && device < kMaxDevices, "device index %d is outside the static scratch table", device);
    unsigned char* known = static_scratch_of_device[device].load(std::memory_order_acquire);
    if (known == nullptr) {
        void* address = nullptr;
        status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (status != hipSuccess || address == nullptr)
            return fail(KHM_ERR_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(status));
        known = static_cast<unsigned char*>(address);
        static_scratch_of_device[device].store(known, std::memory_order_release);
    }
    *out = known;
    return KHM_OK;
}

extern "C" uint64_t khm_sliced_kv_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int khm_sliced_kv_map_reduce_static(const khm_sliced_kv* compute, const khm_sliced_kv_static_buffers* buffers, khm_buffer gates,
                                               khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                               khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(compute != nullptr && buffers != nullptr, "compute and buffers must not be null");
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    // the region layout: [arrival counters | exp sums | max logits | partial outputs], each 256-byte aligned
    auto aligned = [](uint64_t bytes) { return (bytes + 255) & ~255ull; };
    const uint64_t counter_bytes = khm_sliced_kv_arrival_counters_bytes(&config, &compute->variant, &shape);
    const uint64_t stats_bytes = khm_sliced_kv_partial_output_stats_bytes(&config, &shape);
    const uint64_t partial_bytes = khm_sliced_kv_partial_output_bytes(&config, &shape);
    const uint64_t needed = kStaticCounterBytes + 2 * aligned(stats_bytes) + aligned(partial_bytes);
    KHM_REQUIRE(counter_bytes <= kStaticCounterBytes && needed <= kStaticScratchBytes,
                "shape needs %llu bytes of partial state and %llu bytes of arrival counters; the static scratch holds %llu and %llu: "
                "use khm_sliced_kv_map_reduce with caller buffers",
                (unsigned long long)(needed - kStaticCounterBytes), (unsigned long long)counter_bytes,
                (unsigned long long)(kStaticScratchBytes - kStaticCounterBytes), (unsigned long long)kStaticCounterBytes);
    unsigned char* base = nullptr;
    if (int s = static_scratch_pointer(&base)) return s;
    khm_sliced_kv_map_buffers map_buffers{};
    map_buffers.q = buffers->q;
    map_buffers.kv_pages = buffers->kv_pages;
    map_buffers.req_slots = buffers->req_slots;
    map_buffers.page_ids = buffers->page_ids;
    map_buffers.sdpa_map_task_templates = buffers->sdpa_map_task_templates;
    map_buffers.partial_exp_sums = khm_buffer{base + kStaticCounterBytes, stats_bytes};
    map_buffers.partial_max_logits = khm_buffer{base + kStaticCounterBytes + aligned(stats_bytes), stats_bytes};
    map_buffers.partial_output = khm_buffer{base + kStaticCounterBytes + 2 * aligned(stats_bytes), partial_bytes};
    KHM_BUFFER_AT_LEAST(buffers->cu_sdpa_partial_outputs, ((uint64_t)shape.num_total_tokens + 1) * 4, "cu_sdpa_partial_outputs");
    KHM_BUFFER_AT_LEAST(buffers->output, khm_gqa_sdpa_q_bytes(&config, &shape), "output");
    if (gates.ptr != nullptr) KHM_BUFFER_AT_LEAST(gates, khm_gqa_sdpa_q_bytes(&config, &shape), "gates");
    // The counters must start at zero.  A finished call leaves them zero, but the array is shared by every call on this
    // GPU and an earlier call may have been abandoned half-way, so they are cleared here - by a kernel, not a memset
    // node, so that the call can be captured into a HIP graph.
    const uint32_t counters = (uint32_t)(counter_bytes / 4);
    KHM_LAUNCH(clear_u32_kernel, dim3((counters + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<uint32_t*>(base), counters);
    if (int s = check_launch("static scratch clear")) return s;
    const FusedReduceArgs fused{static_cast<const uint32_t*>(buffers->cu_sdpa_partial_outputs.ptr), reinterpret_cast<uint32_t*>(base),
                                static_cast<uint16_t*>(buffers->output.ptr), static_cast<const uint16_t*>(gates.ptr)};
    return launch_sliced_kv_map(compute, &map_buffers, page_table_index, num_active_tokens, num_active_kv_splits, replay_parameters,
                                stream, &fused);
}

static int launch_sliced_kv_reduce(const khm_sliced_kv* compute, const khm_sliced_kv_reduce_buffers* buffers, const khm_buffer* gates,
                                   khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    KHM_REQUIRE(compute != nullptr && buffers != nullptr, "compute and buffers must not be null");
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    // ReduceInvocation::validate (sliced_kv.rs:651-662)
    if (int s = validate_replay(num_active_tokens, 1, shape.num_total_tokens, replay_parameters, "num_active_tokens")) return s;
    KHM_BUFFER_AT_LEAST(buffers->partial_exp_sums, khm_sliced_kv_partial_output_stats_bytes(&config, &shape), "partial_exp_sums");
    KHM_BUFFER_AT_LEAST(buffers->partial_max_logits, khm_sliced_kv_partial_output_stats_bytes(&config, &shape), "partial_max_logits");
    KHM_BUFFER_AT_LEAST(buffers->partial_output, khm_sliced_kv_partial_output_bytes(&config, &shape), "partial_output");
    KHM_BUFFER_AT_LEAST(buffers->cu_sdpa_partial_outputs, ((uint64_t)shape.num_total_tokens + 1) * 4, "cu_sdpa_partial_outputs");
    KHM_BUFFER_AT_LEAST(buffers->output, khm_gqa_sdpa_q_bytes(&config, &shape), "output");
    if (gates != nullptr) KHM_BUFFER_AT_LEAST(*gates, khm_gqa_sdpa_q_bytes(&config, &shape), "gates");
    ReduceParams p{};
    p.exp_sums = static_cast<const float*>(buffers->partial_exp_sums.ptr);
    p.max_logits = static_cast<const float*>(buffers->partial_max_logits.ptr);
    p.partial = buffers->partial_output.ptr;
    p.q_token_ranges = nullptr;
    p.cu_partial_outputs = static_cast<const uint32_t*>(buffers->cu_sdpa_partial_outputs.ptr);
    p.gates = gates ? static_cast<const uint16_t*>(gates->ptr) : nullptr;
    p.output = static_cast<uint16_t*>(buffers->output.ptr);
    p.replay_parameters = replay_parameters;
    p.num_active = to_device(num_active_tokens);
    p.num_q_heads = config.num_q_heads;
    p.head_dim = config.head_dim;
    p.max_q_tokens = 1;
    p.partial_is_f32 = config.partial_dtype == KHM_DTYPE_F32;
    launch_reduce_kernel(config, shape, false, shape.num_total_tokens, 1, compute->reduce, p, static_cast<hipStream_t>(stream));
    return check_launch("sliced-KV reduce");
}

extern "C" int khm_sliced_kv_reduce(const khm_sliced_kv* compute, const khm_sliced_kv_reduce_buffers* buffers,
                                    khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    return launch_sliced_kv_reduce(compute, buffers, nullptr, num_active_tokens, replay_parameters, stream);
}

extern "C" int khm_sliced_kv_reduce_gated(const khm_sliced_kv* compute, const khm_sliced_kv_reduce_buffers* buffers, khm_buffer gates,
                                          khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    return launch_sliced_kv_reduce(compute, buffers, &gates, num_active_tokens, replay_parameters, stream);
}

// ------------------------------------------------------------------------------------------ sliced-Q

extern "C" int khm_sliced_q_create(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant, const khm_gqa_sdpa_shape* shape,
                                   int direct_output, khm_sliced_q** out) {
    clear_error();
    if (int status = validate_component_config(config, true)) return status;
    KHM_REQUIRE(variant != nullptr && shape != nullptr && out != nullptr, "variant, shape and out must not be null");
    const khm_sdpa_config sdpa = static_config(*config);
    KHM_REQUIRE(variant_supports(*variant, sdpa), "GQA SDPA execution variant does not support the config");
    KHM_REQUIRE(variant->map_kind != KHM_MAP_SLICED_KV, "GQA SplitKV SlicedQ requires a sliced-Q execution variant");
    // Shape::validate (sliced_q.rs:255-273)
    KHM_REQUIRE(shape->num_total_tokens > 0, "GQA SplitKV SlicedQ shape requires tokens");
    KHM_REQUIRE(shape->num_total_q_token_tiles > 0 && shape->num_total_q_token_tiles <= shape->num_total_tokens,
                "GQA SplitKV SlicedQ Q-token tiles must be in 1..=num_total_tokens");
    KHM_REQUIRE(shape->num_total_sdpa_map_task_templates >= shape->num_total_q_token_tiles,
                "GQA SplitKV SlicedQ needs at least one Map task template per Q-token tile");
    KHM_REQUIRE(!mul_overflows_u32(shape->num_total_q_token_tiles, 2),
                "GQA SplitKV SlicedQ Q-token-range metadata exceeds the shader u32 element-index domain");
    KHM_REQUIRE(!mul_overflows_u32(shape->num_total_tokens, 2),
                "GQA SplitKV SlicedQ visible K/V-token-range metadata exceeds the shader u32 element-index domain");
    KHM_REQUIRE(!mul_overflows_u32(shape->num_total_sdpa_map_task_templates, 3),
                "GQA SplitKV SlicedQ map TaskTemplate metadata exceeds the shader u32 element-index domain");
    std::string why;
    const int family = kernel_family(sdpa, *variant, config->kv_dtype, &why);
    if (family == 0) return fail(KHM_ERR_UNSUPPORTED, "%s", why.c_str());
    auto* compute = new khm_sliced_q();
    compute->config = *config;
    compute->variant = *variant;
    compute->shape = *shape;
    compute->tokens_per_page = sdpa.tokens_per_page;
    compute->num_q_head_ranges = div_ceil_u32(sdpa.num_q_heads / sdpa.num_kv_heads, variant->map_max_q_heads);
    compute->direct = direct_output != 0;
    const uint32_t coordinates = variant->map_max_q_tokens * variant->map_max_q_heads;
    if (family == 1) {
        compute->map = select_small_tile_kernel(config->head_dim, div_ceil_u32(coordinates, 16), config->kv_dtype);
        compute->map_threads = kMapWaves * 64;
        compute->map_smem_bytes = 0;
        compute->map_merges_in_kernel = true;
    } else {
        compute->map_merges_in_kernel = false;
        const TileKernelChoice choice = select_tile_kernel(config->head_dim, coordinates, config->kv_dtype, compute->direct);
        compute->map = choice.kernel;
        compute->map_threads = choice.threads;
        compute->map_smem_bytes = choice.smem_bytes;
        if (choice.kernel != nullptr) {
            // more than 64 KB of LDS per block has to be requested once per kernel
            const hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(choice.kernel),
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)choice.smem_bytes);
            if (status != hipSuccess) {
                delete compute;
                return fail(KHM_ERR_HIP, "could not reserve %u bytes of LDS: %s", choice.smem_bytes, hipGetErrorString(status));
            }
        }
    }
    compute->reduce = select_reduce_kernel(config->head_dim, true);
    if (compute->map == nullptr || compute->reduce == nullptr) {
        delete compute;
        return fail(KHM_ERR_UNSUPPORTED, "no gfx950 sliced-Q kernel for head_dim %u", config->head_dim);
    }
    *out = compute;
    return KHM_OK;
}

extern "C" void khm_sliced_q_destroy(khm_sliced_q* compute) { delete compute; }
extern "C" const void* khm_sliced_q_map_kernel_id(const khm_sliced_q* compute) { return reinterpret_cast<const void*>(compute->map); }

static int launch_sliced_q_map(const khm_sliced_q* compute, const khm_buffer& q, const khm_buffer& kv_pages, const khm_buffer& req_slots,
                               const khm_buffer& page_ids, const khm_buffer& visible, const khm_buffer& ranges,
                               const khm_buffer& templates, const khm_buffer* partial, const khm_buffer* sums,
                               const khm_buffer* maxs, const khm_buffer* output, khm_replay_u32 page_table_index,
                               khm_replay_u32 num_active_tokens, khm_replay_u32 num_active_q_token_tiles,
                               khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream,
                               const FusedReduceArgs* fused = nullptr, const khm_buffer* direct_gates = nullptr) {
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    // MapInvocation::validate / DirectInvocation::validate (sliced_q.rs:519-545)
    if (int s = validate_replay(page_table_index, 0, config.page_table_layout.num_gqa_layers - 1, replay_parameters, "page_table_index")) return s;
    if (int s = validate_replay(num_active_tokens, 1, shape.num_total_tokens, replay_parameters, "num_active_tokens")) return s;
    if (int s = validate_replay(num_active_q_token_tiles, 1, shape.num_total_q_token_tiles, replay_parameters, "num_active_q_token_tiles")) return s;
    if (int s = validate_replay(num_active_kv_splits, 0, shape.num_total_sdpa_map_task_templates, replay_parameters, "num_active_kv_splits")) return s;
    KHM_BUFFER_AT_LEAST(q, khm_gqa_sdpa_q_bytes(&config, &shape), "q");
    KHM_BUFFER_AT_LEAST(kv_pages, config.page_bytes, "kv_pages");
    KHM_BUFFER_AT_LEAST(req_slots, (uint64_t)shape.num_total_tokens * 4, "req_slots");
    KHM_BUFFER_AT_LEAST(page_ids, khm_gqa_sdpa_page_ids_bytes(&config), "page_ids");
    KHM_BUFFER_AT_LEAST(visible, (uint64_t)shape.num_total_tokens * 8, "visible_kv_token_ranges");
    KHM_BUFFER_AT_LEAST(ranges, (uint64_t)shape.num_total_q_token_tiles * 8, "q_token_ranges");
    KHM_BUFFER_AT_LEAST(templates, (uint64_t)shape.num_total_sdpa_map_task_templates * 12, "sdpa_map_task_templates");
    MapParams p{};
    if (output != nullptr) {
        KHM_BUFFER_AT_LEAST(*output, khm_gqa_sdpa_q_bytes(&config, &shape), "output");
        p.out = output->ptr;
        p.output_mode = kMapDirectBf16;
        if (direct_gates != nullptr) {
            KHM_BUFFER_AT_LEAST(*direct_gates, khm_gqa_sdpa_q_bytes(&config, &shape), "gates");
            p.gates = static_cast<const uint16_t*>(direct_gates->ptr);
        }
    } else {
        KHM_BUFFER_AT_LEAST(*partial, khm_sliced_q_partial_output_bytes(&config, &compute->variant, &shape), "partial_output");
        KHM_BUFFER_AT_LEAST(*sums, khm_sliced_q_partial_output_stats_bytes(&config, &compute->variant, &shape), "partial_exp_sums");
        KHM_BUFFER_AT_LEAST(*maxs, khm_sliced_q_partial_output_stats_bytes(&config, &compute->variant, &shape), "partial_max_logits");
        p.out = partial->ptr;
        p.exp_sums = static_cast<float*>(sums->ptr);
        p.max_logits = static_cast<float*>(maxs->ptr);
        p.output_mode = config.partial_dtype == KHM_DTYPE_F32 ? kMapPartialF32 : kMapPartialBf16;
    }
    p.q = static_cast<const uint16_t*>(q.ptr);
    p.kv_pages = static_cast<const uint8_t*>(kv_pages.ptr);
    p.req_slots = static_cast<const uint32_t*>(req_slots.ptr);
    p.page_ids = static_cast<const uint32_t*>(page_ids.ptr);
    p.visible_ranges = static_cast<const uint32_t*>(visible.ptr);
    p.q_token_ranges = static_cast<const uint32_t*>(ranges.ptr);
    p.templates = static_cast<const uint32_t*>(templates.ptr);
    p.replay_parameters = replay_parameters;
    p.layer_index = to_device(page_table_index);
    p.num_active_tokens = to_device(num_active_tokens);
    p.num_active_q_token_tiles = to_device(num_active_q_token_tiles);
    p.num_active_kv_splits = to_device(num_active_kv_splits);
    fill_map_geometry(*compute, &p);
    if (fused != nullptr) {
        p.cu_partial_outputs = fused->cu_partial_outputs;
        p.arrival_counters = fused->arrival_counters;
        p.final_output = fused->final_output;
        p.gates = fused->gates;
    }
    const dim3 grid(shape.num_total_sdpa_map_task_templates, config.num_kv_heads * compute->num_q_head_ranges, 1);
    KHM_LAUNCH(compute->map, grid, dim3(compute->map_threads), compute->map_smem_bytes, static_cast<hipStream_t>(stream), p);
    return check_launch("sliced-Q map");
}

extern "C" uint64_t khm_sliced_q_arrival_counters_bytes(const khm_gqa_sdpa_config* config, const khm_sdpa_variant* variant,
                                                        const khm_gqa_sdpa_shape* shape) {
    const uint32_t ranges = div_ceil_u32(config->num_q_heads / config->num_kv_heads, variant->map_max_q_heads);
    return (uint64_t)shape->num_total_q_token_tiles * config->num_kv_heads * ranges * 4;
}

extern "C" int khm_sliced_q_map_reduce(const khm_sliced_q* compute, const khm_sliced_q_map_buffers* map_buffers,
                                       const khm_sliced_q_reduce_buffers* reduce_buffers, khm_buffer arrival_counters,
                                       khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                       khm_replay_u32 num_active_q_token_tiles, khm_replay_u32 num_active_kv_splits,
                                       const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(compute != nullptr && map_buffers != nullptr && reduce_buffers != nullptr, "compute and buffers must not be null");
    KHM_REQUIRE(!compute->direct, "GQA SplitKV SlicedQ direct-output compute cannot record a partial Map");
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    KHM_REQUIRE(reduce_buffers->partial_output.ptr == map_buffers->partial_output.ptr &&
                    reduce_buffers->partial_exp_sums.ptr == map_buffers->partial_exp_sums.ptr &&
                    reduce_buffers->partial_max_logits.ptr == map_buffers->partial_max_logits.ptr &&
                    reduce_buffers->q_token_ranges.ptr == map_buffers->q_token_ranges.ptr,
                "fused Map/Reduce needs the same partial and Q-token-range buffers on both sides");
    KHM_BUFFER_AT_LEAST(reduce_buffers->cu_sdpa_partial_outputs, ((uint64_t)shape.num_total_q_token_tiles + 1) * 4, "cu_sdpa_partial_outputs");
    KHM_BUFFER_AT_LEAST(reduce_buffers->output, khm_gqa_sdpa_q_bytes(&config, &shape), "output");
    KHM_BUFFER_AT_LEAST(arrival_counters, khm_sliced_q_arrival_counters_bytes(&config, &compute->variant, &shape), "arrival_counters");
    if (!compute->map_merges_in_kernel) {
        // the LDS-tiled Map kernel has no merge epilogue: same result from the two launches, in stream order
        if (int s = khm_sliced_q_map(compute, map_buffers, page_table_index, num_active_tokens, num_active_q_token_tiles,
                                     num_active_kv_splits, replay_parameters, stream))
            return s;
        return khm_sliced_q_reduce(compute, reduce_buffers, num_active_q_token_tiles, replay_parameters, stream);
    }
    const FusedReduceArgs fused{static_cast<const uint32_t*>(reduce_buffers->cu_sdpa_partial_outputs.ptr),
                                static_cast<uint32_t*>(arrival_counters.ptr), static_cast<uint16_t*>(reduce_buffers->output.ptr), nullptr};
    return launch_sliced_q_map(compute, map_buffers->q, map_buffers->kv_pages, map_buffers->req_slots, map_buffers->page_ids,
                               map_buffers->visible_kv_token_ranges, map_buffers->q_token_ranges, map_buffers->sdpa_map_task_templates,
                               &map_buffers->partial_output, &map_buffers->partial_exp_sums, &map_buffers->partial_max_logits, nullptr,
                               page_table_index, num_active_tokens, num_active_q_token_tiles, num_active_kv_splits, replay_parameters,
                               stream, &fused);
}

extern "C" int khm_sliced_q_map(const khm_sliced_q* compute, const khm_sliced_q_map_buffers* buffers, khm_replay_u32 page_table_index,
                                khm_replay_u32 num_active_tokens, khm_replay_u32 num_active_q_token_tiles,
                                khm_replay_u32 num_active_kv_splits, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(compute != nullptr && buffers != nullptr, "compute and buffers must not be null");
    KHM_REQUIRE(!compute->direct, "GQA SplitKV SlicedQ direct-output compute cannot record a partial Map");
    return launch_sliced_q_map(compute, buffers->q, buffers->kv_pages, buffers->req_slots, buffers->page_ids,
                               buffers->visible_kv_token_ranges, buffers->q_token_ranges, buffers->sdpa_map_task_templates,
                               &buffers->partial_output, &buffers->partial_exp_sums, &buffers->partial_max_logits, nullptr,
                               page_table_index, num_active_tokens, num_active_q_token_tiles, num_active_kv_splits,
                               replay_parameters, stream);
}

static int sliced_q_direct(const khm_sliced_q* compute, const khm_sliced_q_direct_buffers* buffers, const khm_buffer* gates,
                           khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                           khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(compute != nullptr && buffers != nullptr, "compute and buffers must not be null");
    KHM_REQUIRE(compute->direct, "GQA SplitKV SlicedQ direct output requires a direct-output compute");
    // One direct Map owns each Q range: both padded domains have the same extent (sdpa.rs:564-568).
    KHM_REQUIRE(compute->shape.num_total_sdpa_map_task_templates == compute->shape.num_total_q_token_tiles,
                "GQA direct output requires one Map task template per Q-token tile");
    return launch_sliced_q_map(compute, buffers->q, buffers->kv_pages, buffers->req_slots, buffers->page_ids,
                               buffers->visible_kv_token_ranges, buffers->q_token_ranges, buffers->sdpa_map_task_templates, nullptr,
                               nullptr, nullptr, &buffers->output, page_table_index, num_active_tokens, num_active_q_token_tiles,
                               num_active_q_token_tiles, replay_parameters, stream, nullptr, gates);
}

extern "C" int khm_sliced_q_direct(const khm_sliced_q* compute, const khm_sliced_q_direct_buffers* buffers,
                                   khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                   khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream) {
    return sliced_q_direct(compute, buffers, nullptr, page_table_index, num_active_tokens, num_active_q_token_tiles, replay_parameters, stream);
}

extern "C" int khm_sliced_q_direct_gated(const khm_sliced_q* compute, const khm_sliced_q_direct_buffers* buffers, khm_buffer gates,
                                         khm_replay_u32 page_table_index, khm_replay_u32 num_active_tokens,
                                         khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream) {
    return sliced_q_direct(compute, buffers, &gates, page_table_index, num_active_tokens, num_active_q_token_tiles, replay_parameters, stream);
}

static int sliced_q_reduce(const khm_sliced_q* compute, const khm_sliced_q_reduce_buffers* buffers, const khm_buffer* gates,
                           khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(compute != nullptr && buffers != nullptr, "compute and buffers must not be null");
    KHM_REQUIRE(!compute->direct, "GQA SplitKV SlicedQ direct-output compute has no Reduce");
    const khm_gqa_sdpa_config& config = compute->config;
    const khm_gqa_sdpa_shape& shape = compute->shape;
    // ReduceInvocation::validate (sliced_q.rs:603-618)
    if (int s = validate_replay(num_active_q_token_tiles, 1, shape.num_total_q_token_tiles, replay_parameters, "num_active_q_token_tiles")) return s;
    KHM_BUFFER_AT_LEAST(buffers->partial_output, khm_sliced_q_partial_output_bytes(&config, &compute->variant, &shape), "partial_output");
    KHM_BUFFER_AT_LEAST(buffers->partial_exp_sums, khm_sliced_q_partial_output_stats_bytes(&config, &compute->variant, &shape), "partial_exp_sums");
    KHM_BUFFER_AT_LEAST(buffers->partial_max_logits, khm_sliced_q_partial_output_stats_bytes(&config, &compute->variant, &shape), "partial_max_logits");
    KHM_BUFFER_AT_LEAST(buffers->q_token_ranges, (uint64_t)shape.num_total_q_token_tiles * 8, "q_token_ranges");
    KHM_BUFFER_AT_LEAST(buffers->cu_sdpa_partial_outputs, ((uint64_t)shape.num_total_q_token_tiles + 1) * 4, "cu_sdpa_partial_outputs");
    KHM_BUFFER_AT_LEAST(buffers->output, khm_gqa_sdpa_q_bytes(&config, &shape), "output");
    ReduceParams p{};
    p.exp_sums = static_cast<const float*>(buffers->partial_exp_sums.ptr);
    p.max_logits = static_cast<const float*>(buffers->partial_max_logits.ptr);
    p.partial = buffers->partial_output.ptr;
    p.q_token_ranges = static_cast<const uint32_t*>(buffers->q_token_ranges.ptr);
    p.cu_partial_outputs = static_cast<const uint32_t*>(buffers->cu_sdpa_partial_outputs.ptr);
    p.gates = nullptr;
    if (gates != nullptr) {
        KHM_BUFFER_AT_LEAST(*gates, khm_gqa_sdpa_q_bytes(&config, &shape), "gates");
        p.gates = static_cast<const uint16_t*>(gates->ptr);
    }
    p.output = static_cast<uint16_t*>(buffers->output.ptr);
    p.replay_parameters = replay_parameters;
    p.num_active = to_device(num_active_q_token_tiles);
    p.num_q_heads = config.num_q_heads;
    p.head_dim = config.head_dim;
    p.max_q_tokens = compute->variant.map_max_q_tokens;
    p.partial_is_f32 = config.partial_dtype == KHM_DTYPE_F32;
    KHM_REQUIRE(!mul_overflows_u32(shape.num_total_q_token_tiles, compute->variant.map_max_q_tokens),
                "GQA SplitKV SlicedQ reduce grid exceeds the u32 domain");
    launch_reduce_kernel(config, shape, true, shape.num_total_q_token_tiles, compute->variant.map_max_q_tokens, compute->reduce, p,
                         static_cast<hipStream_t>(stream));
    return check_launch("sliced-Q reduce");
}

extern "C" int khm_sliced_q_reduce(const khm_sliced_q* compute, const khm_sliced_q_reduce_buffers* buffers,
                                   khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream) {
    return sliced_q_reduce(compute, buffers, nullptr, num_active_q_token_tiles, replay_parameters, stream);
}

extern "C" int khm_sliced_q_reduce_gated(const khm_sliced_q* compute, const khm_sliced_q_reduce_buffers* buffers, khm_buffer gates,
                                         khm_replay_u32 num_active_q_token_tiles, const uint32_t* replay_parameters, void* stream) {
    return sliced_q_reduce(compute, buffers, &gates, num_active_q_token_tiles, replay_parameters, stream);
}

// ------------------------------------------------------------------------------------------ gate

extern "C" int khm_gqa_activation_gate(uint32_t dtype, uint32_t num_q_heads, uint32_t head_dim, uint32_t num_total_tokens,
                                       khm_buffer attention_output, khm_buffer gates, khm_buffer output,
                                       khm_replay_u32 num_active_tokens, const uint32_t* replay_parameters, void* stream) {
    clear_error();
    KHM_REQUIRE(dtype == KHM_DTYPE_F32 || dtype == KHM_DTYPE_BF16, "unsupported GQA activation gate dtype");
    KHM_REQUIRE(num_q_heads > 0 && head_dim > 0 && num_total_tokens > 0, "GQA activation/gate requires tokens, heads and a head dimension");
    KHM_REQUIRE(!mul_overflows_u32(num_total_tokens, num_q_heads, head_dim), "GQA activation/gate exceeds the shader u32 count domain");
    if (int s = validate_replay(num_active_tokens, 1, num_total_tokens, replay_parameters, "num_active_tokens")) return s;
    const uint64_t values = (uint64_t)num_total_tokens * num_q_heads * head_dim;
    const uint64_t bytes = values * dtype_item_size(dtype);
    KHM_BUFFER_AT_LEAST(attention_output, bytes, "attention_output");
    KHM_BUFFER_AT_LEAST(gates, bytes, "gates");
    KHM_BUFFER_AT_LEAST(output, bytes, "output");
    GateParams p{};
    p.attention = attention_output.ptr;
    p.gates = gates.ptr;
    p.output = output.ptr;
    p.replay_parameters = replay_parameters;
    p.num_active_tokens = to_device(num_active_tokens);
    p.values_per_token = num_q_heads * head_dim;
    p.is_f32 = dtype == KHM_DTYPE_F32;
    const uintptr_t address_bits = reinterpret_cast<uintptr_t>(attention_output.ptr) | reinterpret_cast<uintptr_t>(gates.ptr) |
                                   reinterpret_cast<uintptr_t>(output.ptr);
    if (address_bits % 16 == 0) {
        const uint64_t per_block = 256ull * gate_elements_per_thread(p.is_f32 != 0);
        const uint32_t blocks = (uint32_t)((values + per_block - 1) / per_block);
        if (p.is_f32) KHM_LAUNCH(activation_gate_vector_kernel<true>, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), p);
        else KHM_LAUNCH(activation_gate_vector_kernel<false>, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), p);
        return check_launch("activation gate");
    }
    const uint32_t blocks = (uint32_t)((values + 255) / 256);
    KHM_LAUNCH(activation_gate_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return check_launch("activation gate");
}
