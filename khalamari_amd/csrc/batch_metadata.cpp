// GPU metadata ABI of one SDPA batch: per-token request slots, request-absolute token indices and
// visible KV ranges, Q-token ranges, map task templates (padded with u32::MAX) and cumulative partial
// counts.  Behaviour follows GQAMetadataBuffers::{new, update}
// (crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:98-253): which arrays are written, how far,
// and what is left untouched.  The reference writes unified-memory buffers in place; here the values are
// staged in pinned host memory and copied to device arrays on the caller's stream.
#include <hip/hip_runtime.h>

#include <vector>

#include "common.h"

using namespace khm;

struct khm_selection;
extern "C" {
int khm_selection_variant(const khm_selection*, khm_sdpa_variant*);
int khm_selection_replay_shape(const khm_selection*, khm_gqa_replay_shape*);
uint32_t khm_selection_num_q_token_ranges(const khm_selection*);
uint32_t khm_selection_num_map_task_templates(const khm_selection*);
int khm_selection_q_token_ranges(const khm_selection*, khm_q_token_range*, uint32_t);
int khm_selection_map_task_templates(const khm_selection*, khm_map_task_template*, uint32_t);
int khm_selection_cu_partial_outputs(const khm_selection*, uint32_t*, uint32_t);
}

namespace khm {

constexpr int kNumArrays = 6;

struct MetadataCounts {
    uint64_t written[kNumArrays];  // u32 values written per array by one update
};

// Shared by the device-backed update and the pure host form.
static int compute_metadata(const uint32_t* req_slots, const uint32_t* token_indices, const uint32_t* cu_tokens, uint32_t num_requests,
                            const khm_selection* selection, uint64_t token_capacity, uint64_t template_capacity, uint32_t* const out[kNumArrays],
                            MetadataCounts* counts, khm_gqa_replay_shape* shape_out) {
    KHM_REQUIRE(selection != nullptr, "GQA batch metadata requires a selection");
    KHM_REQUIRE(req_slots != nullptr && token_indices != nullptr && cu_tokens != nullptr, "GQA batch arrays must not be null");
    KHM_REQUIRE(cu_tokens[0] == 0, "GQA batch cu_tokens must start at zero");
    khm_gqa_replay_shape shape;
    khm_selection_replay_shape(selection, &shape);
    KHM_REQUIRE(cu_tokens[num_requests] == shape.num_tokens, "GQA batch cu_tokens must end at the selection's token count");
    KHM_REQUIRE(shape.num_total_tokens <= token_capacity, "GQA replay tokens exceed the metadata capacity");
    KHM_REQUIRE(shape.num_total_q_token_tiles <= token_capacity, "GQA replay Q-token tiles exceed the metadata capacity");
    KHM_REQUIRE(shape.num_total_sdpa_map_task_templates <= template_capacity, "GQA replay Map task templates exceed the metadata capacity");
    khm_sdpa_variant variant;
    khm_selection_variant(selection, &variant);

    uint64_t t = 0;
    for (uint32_t r = 0; r < num_requests; ++r) {
        KHM_REQUIRE(cu_tokens[r] <= cu_tokens[r + 1], "GQA batch cu_tokens must be nondecreasing");
        const uint32_t n = cu_tokens[r + 1] - cu_tokens[r];
        KHM_REQUIRE((uint64_t)token_indices[r] + n <= 0xffffffffull, "GQA request context length must fit u32");
        for (uint32_t i = 0; i < n; ++i, ++t) {
            const uint32_t flat_token_index = token_indices[r] + i;
            out[KHM_METADATA_REQ_SLOTS][t] = req_slots[r];
            out[KHM_METADATA_FLAT_TOKEN_INDICES][t] = flat_token_index;
            out[KHM_METADATA_VISIBLE_KV_TOKEN_RANGES][2 * t] = 0;
            out[KHM_METADATA_VISIBLE_KV_TOKEN_RANGES][2 * t + 1] = flat_token_index + 1;
        }
    }
    KHM_REQUIRE(t == shape.num_tokens, "GQA batch token count must match the selection");
    counts->written[KHM_METADATA_REQ_SLOTS] = t;
    counts->written[KHM_METADATA_FLAT_TOKEN_INDICES] = t;
    counts->written[KHM_METADATA_VISIBLE_KV_TOKEN_RANGES] = 2 * t;

    const uint32_t num_ranges = khm_selection_num_q_token_ranges(selection);
    KHM_REQUIRE(num_ranges == shape.num_q_token_tiles, "GQA selection Q-token ranges must match its replay shape");
    counts->written[KHM_METADATA_Q_TOKEN_RANGES] = 0;
    if (variant.map_kind != KHM_MAP_SLICED_KV) {
        std::vector<khm_q_token_range> ranges(num_ranges);
        khm_selection_q_token_ranges(selection, ranges.data(), num_ranges);
        for (uint32_t i = 0; i < num_ranges; ++i) {
            out[KHM_METADATA_Q_TOKEN_RANGES][2 * (uint64_t)i] = ranges[i].flat_q_token_begin;
            out[KHM_METADATA_Q_TOKEN_RANGES][2 * (uint64_t)i + 1] = ranges[i].flat_q_token_end;
        }
        counts->written[KHM_METADATA_Q_TOKEN_RANGES] = 2 * (uint64_t)num_ranges;
    }

    const uint32_t num_templates = khm_selection_num_map_task_templates(selection);
    KHM_REQUIRE(num_templates == shape.num_sdpa_map_task_templates, "GQA selection templates must match its replay shape");
    std::vector<khm_map_task_template> templates(num_templates);
    khm_selection_map_task_templates(selection, templates.data(), num_templates);
    uint32_t* template_out = out[KHM_METADATA_SDPA_MAP_TASK_TEMPLATES];
    for (uint32_t i = 0; i < num_templates; ++i) {
        template_out[3 * (uint64_t)i] = templates[i].q_token_range_index;
        template_out[3 * (uint64_t)i + 1] = templates[i].kv_token_begin;
        template_out[3 * (uint64_t)i + 2] = templates[i].kv_token_end;
    }
    for (uint64_t i = 3 * (uint64_t)num_templates; i < 3 * (uint64_t)shape.num_total_sdpa_map_task_templates; ++i) template_out[i] = 0xffffffffu;
    counts->written[KHM_METADATA_SDPA_MAP_TASK_TEMPLATES] = 3 * (uint64_t)shape.num_total_sdpa_map_task_templates;

    khm_selection_cu_partial_outputs(selection, out[KHM_METADATA_CU_SDPA_PARTIAL_OUTPUTS], num_ranges + 1);
    counts->written[KHM_METADATA_CU_SDPA_PARTIAL_OUTPUTS] = (uint64_t)num_ranges + 1;
    if (shape_out) *shape_out = shape;
    return KHM_OK;
}

}  // namespace khm

struct khm_gqa_metadata {
    uint64_t max_tokens = 0;
    uint64_t max_map_task_templates = 0;
    uint64_t capacity[kNumArrays] = {};  // u32 values
    uint32_t* host[kNumArrays] = {};     // pinned
    uint32_t* device[kNumArrays] = {};
};

extern "C" void khm_gqa_metadata_destroy(khm_gqa_metadata* metadata) {
    if (metadata == nullptr) return;
    for (int i = 0; i < kNumArrays; ++i) {
        if (metadata->host[i]) (void)hipHostFree(metadata->host[i]);
        if (metadata->device[i]) (void)hipFree(metadata->device[i]);
    }
    delete metadata;
}

extern "C" int khm_gqa_metadata_create(uint64_t max_tokens, uint64_t max_map_task_templates, khm_gqa_metadata** out) {
    clear_error();
    KHM_REQUIRE(out != nullptr, "metadata output must not be null");
    KHM_REQUIRE(max_tokens > 0, "GQA batch metadata requires tokens");
    KHM_REQUIRE(max_tokens <= 0xffffffffull, "GQA token capacity must fit u32");
    KHM_REQUIRE(max_map_task_templates > 0, "GQA batch metadata requires Map task templates");
    KHM_REQUIRE(max_map_task_templates <= 0xffffffffull, "GQA Map task-template capacity must fit u32");
    auto* metadata = new khm_gqa_metadata();
    metadata->max_tokens = max_tokens;
    metadata->max_map_task_templates = max_map_task_templates;
    metadata->capacity[KHM_METADATA_REQ_SLOTS] = max_tokens;
    metadata->capacity[KHM_METADATA_FLAT_TOKEN_INDICES] = max_tokens;
    metadata->capacity[KHM_METADATA_VISIBLE_KV_TOKEN_RANGES] = max_tokens * 2;
    metadata->capacity[KHM_METADATA_Q_TOKEN_RANGES] = max_tokens * 2;
    metadata->capacity[KHM_METADATA_SDPA_MAP_TASK_TEMPLATES] = max_map_task_templates * 3;
    metadata->capacity[KHM_METADATA_CU_SDPA_PARTIAL_OUTPUTS] = max_tokens + 1;
    for (int i = 0; i < kNumArrays; ++i) {
        const size_t bytes = metadata->capacity[i] * sizeof(uint32_t);
        hipError_t status = hipHostMalloc(reinterpret_cast<void**>(&metadata->host[i]), bytes, hipHostMallocDefault);
        if (status == hipSuccess) status = hipMalloc(reinterpret_cast<void**>(&metadata->device[i]), bytes);
        if (status == hipSuccess) status = hipMemset(metadata->device[i], 0, bytes);  // new_zeroed_elements
        if (status != hipSuccess) {
            khm_gqa_metadata_destroy(metadata);
            return fail(KHM_ERR_HIP, "GQA batch metadata allocation failed: %s", hipGetErrorString(status));
        }
        __builtin_memset(metadata->host[i], 0, bytes);
    }
    *out = metadata;
    return KHM_OK;
}

extern "C" int khm_gqa_metadata_update(khm_gqa_metadata* metadata, const uint32_t* req_slots, const uint32_t* token_indices,
                                       const uint32_t* cu_tokens, uint32_t num_requests, const khm_selection* selection, void* stream,
                                       khm_gqa_replay_shape* out_shape) {
    clear_error();
    KHM_REQUIRE(metadata != nullptr, "metadata must not be null");
    MetadataCounts counts{};
    // The pinned staging arrays are reused by every update: wait until earlier copies have drained.
    hipError_t status = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (status != hipSuccess) return fail(KHM_ERR_HIP, "GQA batch metadata stream wait failed: %s", hipGetErrorString(status));
    if (int result = compute_metadata(req_slots, token_indices, cu_tokens, num_requests, selection, metadata->max_tokens,
                                      metadata->max_map_task_templates, metadata->host, &counts, out_shape))
        return result;
    for (int i = 0; i < kNumArrays; ++i) {
        if (counts.written[i] == 0) continue;
        status = hipMemcpyAsync(metadata->device[i], metadata->host[i], counts.written[i] * sizeof(uint32_t), hipMemcpyHostToDevice,
                                static_cast<hipStream_t>(stream));
        if (status != hipSuccess) return fail(KHM_ERR_HIP, "GQA batch metadata upload failed: %s", hipGetErrorString(status));
    }
    return KHM_OK;
}

extern "C" int khm_gqa_metadata_buffer(const khm_gqa_metadata* metadata, uint32_t which, khm_buffer* out) {
    clear_error();
    KHM_REQUIRE(metadata != nullptr && out != nullptr && which < (uint32_t)kNumArrays, "unknown GQA metadata array");
    out->ptr = metadata->device[which];
    out->len_bytes = metadata->capacity[which] * sizeof(uint32_t);
    return KHM_OK;
}

extern "C" int khm_gqa_metadata_host(const khm_gqa_metadata* metadata, uint32_t which, const uint32_t** out, uint64_t* count) {
    clear_error();
    KHM_REQUIRE(metadata != nullptr && out != nullptr && count != nullptr && which < (uint32_t)kNumArrays, "unknown GQA metadata array");
    *out = metadata->host[which];
    *count = metadata->capacity[which];
    return KHM_OK;
}

extern "C" int khm_gqa_metadata_compute(const uint32_t* req_slots, const uint32_t* token_indices, const uint32_t* cu_tokens,
                                        uint32_t num_requests, const khm_selection* selection, uint32_t* req_slots_by_token,
                                        uint32_t* flat_token_indices, uint32_t* visible_kv_token_ranges, uint32_t* q_token_ranges,
                                        uint32_t* sdpa_map_task_templates, uint32_t* cu_sdpa_partial_outputs, uint64_t token_capacity,
                                        uint64_t template_capacity) {
    clear_error();
    uint32_t* const arrays[kNumArrays] = {req_slots_by_token,    flat_token_indices,      visible_kv_token_ranges,
                                          q_token_ranges,        sdpa_map_task_templates, cu_sdpa_partial_outputs};
    for (uint32_t* array : arrays) KHM_REQUIRE(array != nullptr, "GQA metadata output arrays must not be null");
    MetadataCounts counts{};
    return compute_metadata(req_slots, token_indices, cu_tokens, num_requests, selection, token_capacity, template_capacity, arrays, &counts,
                            nullptr);
}
