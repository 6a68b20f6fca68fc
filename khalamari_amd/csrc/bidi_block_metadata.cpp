// Host logic of the block (DFlash2 proposal) attention path: capacity, execution selection and the GPU metadata of
// "history split-KV partials + one dense block partial" per Q-token range.  Pure integer work, no device calls.
//
// Follows BiDiBlockCapacity / BiDiBlockGQAMetadata::new (crates/inference-executor-core/src/attn/gqa/bidi_block_gqa_core.rs:27-139),
// BiDiBlockGQACapacity::new (crates/inference-executor-metal/src/attn/bidi_block_gqa/capacity.rs:16-48),
// Selector::select (.../bidi_block_gqa/sdpa.rs:46-110) and build_metal_metadata / allocate_history_kv_splits /
// update_with_active_requests (.../bidi_block_gqa/metadata.rs:87-147,182-375).
#include <algorithm>
#include <queue>
#include <tuple>
#include <vector>

#include "common.h"

using namespace khm;

namespace khm {

static bool next_power_of_two_u64(uint64_t value, uint64_t* out) {
    uint64_t power = 1;
    while (power < value) {
        if (power > (UINT64_MAX >> 1)) return false;
        power <<= 1;
    }
    *out = power;
    return true;
}

static int make_capacity(uint64_t max_requests, uint64_t block_size, uint32_t max_q_tokens, khm_bidi_block_capacity* out) {
    // BiDiBlockCapacity::new + validate (bidi_block_gqa_core.rs:35-63)
    KHM_REQUIRE(max_requests > 0, "BiDiBlockGQA capacity requires requests");
    KHM_REQUIRE(block_size > 0, "BiDiBlockGQA capacity requires block tokens");
    const __uint128_t max_tokens = (__uint128_t)max_requests * block_size;
    KHM_REQUIRE(max_tokens <= 0xffffffffull, "BiDiBlockGQA token capacity must fit u32");
    // BiDiBlockGQACapacity::new (capacity.rs:16-48)
    KHM_REQUIRE(max_q_tokens > 0, "BiDiBlockGQA Q-token range must contain tokens");
    const uint64_t ranges_per_request = (block_size + max_q_tokens - 1) / max_q_tokens;
    const uint64_t max_q_token_ranges = max_requests * ranges_per_request;
    const uint64_t min_templates = std::max<uint64_t>((uint64_t)max_tokens, max_q_token_ranges * 2);
    uint64_t max_templates = 0;
    KHM_REQUIRE(next_power_of_two_u64(min_templates, &max_templates) && max_templates <= 0xffffffffull,
                "BiDiBlockGQA Map task-template capacity must fit u32");
    out->max_requests = (uint32_t)max_requests;
    out->block_size = (uint32_t)block_size;
    out->max_tokens = (uint32_t)max_tokens;
    out->max_q_tokens = max_q_tokens;
    out->max_q_token_ranges = (uint32_t)max_q_token_ranges;
    out->max_sdpa_map_task_templates = (uint32_t)max_templates;
    out->max_sdpa_partial_state_groups = max_templates * max_q_tokens;
    return KHM_OK;
}

// allocate_history_kv_splits (metadata.rs:343-371): one split per Q range, then the spare templates go to the range
// with the most iterations per split; ties go to the later range (max-heap on (iterations, index)).
static std::vector<uint64_t> allocate_history_kv_splits(const std::vector<uint64_t>& iterations, uint64_t max_templates) {
    if (iterations.size() == 1) return {std::min(iterations[0], max_templates)};
    std::vector<uint64_t> splits(iterations.size(), 1);
    if (splits.size() == max_templates) return splits;
    std::priority_queue<std::pair<uint64_t, uint64_t>> candidates;
    for (uint64_t index = 0; index < iterations.size(); ++index)
        if (iterations[index] > 1) candidates.emplace(iterations[index], index);
    for (uint64_t used = splits.size(); used < max_templates; ++used) {
        if (candidates.empty()) break;
        const uint64_t index = candidates.top().second;
        candidates.pop();
        ++splits[index];
        if (splits[index] < iterations[index]) candidates.emplace((iterations[index] + splits[index] - 1) / splits[index], index);
    }
    return splits;
}

}  // namespace khm

extern "C" int khm_bidi_block_capacity_new(uint32_t max_requests, uint32_t block_size, uint32_t max_q_tokens, khm_bidi_block_capacity* out) {
    clear_error();
    KHM_REQUIRE(out != nullptr, "out must not be null");
    return make_capacity(max_requests, block_size, max_q_tokens, out);
}

extern "C" int khm_bidi_block_select(const khm_sdpa_config* config, uint32_t max_requests, uint32_t block_size, khm_sdpa_variant* variant,
                                     khm_bidi_block_capacity* capacity) {
    clear_error();
    KHM_REQUIRE(config != nullptr && variant != nullptr && capacity != nullptr, "config, variant and capacity must not be null");
    khm_sdpa_variant variants[16];
    uint32_t count = 0;
    if (int status = khm_sdpa_registry_new(config, variants, 16, &count)) return status;
    KHM_REQUIRE(count > 0, "GQA SDPA registry must contain an execution variant");
    const uint64_t q_heads_per_kv_head = config->num_q_heads / config->num_kv_heads;
    // min_by_key over (K/V load multiplicity, Reverse(kv tokens per iteration), padded Q tokens, partial-state groups,
    // Reverse(max Q heads)); the first minimum wins (sdpa.rs:58-76)
    typedef std::tuple<uint64_t, int64_t, uint64_t, uint64_t, int64_t> Key;
    bool have = false;
    Key best_key;
    for (uint32_t i = 0; i < count; ++i) {
        khm_bidi_block_capacity candidate;
        if (int status = make_capacity(max_requests, block_size, variants[i].map_max_q_tokens, &candidate)) return status;
        const uint64_t ranges_per_request = ((uint64_t)block_size + candidate.max_q_tokens - 1) / candidate.max_q_tokens;
        const uint64_t head_ranges = (q_heads_per_kv_head + variants[i].map_max_q_heads - 1) / variants[i].map_max_q_heads;
        const Key key(ranges_per_request * head_ranges, -(int64_t)variants[i].map_kv_tokens_per_iteration,
                      ranges_per_request * candidate.max_q_tokens, candidate.max_sdpa_partial_state_groups,
                      -(int64_t)variants[i].map_max_q_heads);
        if (!have || key < best_key) {
            have = true;
            best_key = key;
            *variant = variants[i];
            *capacity = candidate;
        }
    }
    return KHM_OK;
}

extern "C" int khm_bidi_block_metadata_compute(const uint32_t* req_slots, uint32_t num_requests, const uint32_t* flat_query_token_indices,
                                               const uint32_t* history_token_begins, const uint32_t* history_token_ends, uint32_t block_size,
                                               const khm_sdpa_variant* variant, uint32_t max_sdpa_map_task_templates,
                                               uint32_t num_active_requests, uint32_t* req_slots_by_token, uint32_t* flat_token_indices,
                                               uint32_t* visible_kv_token_ranges, uint32_t* q_token_ranges,
                                               uint32_t* sdpa_map_task_templates, uint32_t* cu_sdpa_partial_outputs,
                                               khm_gqa_replay_shape* out_shape) {
    clear_error();
    KHM_REQUIRE(req_slots != nullptr && flat_query_token_indices != nullptr && history_token_begins != nullptr && history_token_ends != nullptr,
                "BiDiBlockGQA metadata inputs must not be null");
    KHM_REQUIRE(variant != nullptr && out_shape != nullptr, "variant and out_shape must not be null");
    KHM_REQUIRE(req_slots_by_token != nullptr && flat_token_indices != nullptr && visible_kv_token_ranges != nullptr && q_token_ranges != nullptr &&
                    sdpa_map_task_templates != nullptr && cu_sdpa_partial_outputs != nullptr,
                "BiDiBlockGQA metadata outputs must not be null");
    // BiDiBlockGQAMetadata::new (bidi_block_gqa_core.rs:77-139)
    KHM_REQUIRE(num_requests > 0, "BiDiBlockGQA metadata requires requests");
    KHM_REQUIRE(block_size > 0, "BiDiBlockGQA metadata requires block tokens");
    const uint64_t num_tokens = (uint64_t)num_requests * block_size;
    KHM_REQUIRE(num_tokens <= 0xffffffffull, "BiDiBlockGQA token count must fit u32");
    for (uint32_t i = 0; i < num_requests; ++i)
        for (uint32_t j = 0; j < i; ++j) KHM_REQUIRE(req_slots[i] != req_slots[j], "BiDiBlockGQA metadata requires unique request slots");
    for (uint64_t t = 0; t < num_tokens; ++t)
        KHM_REQUIRE(history_token_begins[t] < history_token_ends[t], "BiDiBlockGQA visible history token ranges must be nonempty half-open ranges");
    // update_with_active_requests (metadata.rs:91-103)
    KHM_REQUIRE(num_active_requests > 0 && num_active_requests <= num_requests,
                "active BiDiBlockGQA requests must fit the materialized request capacity");
    const uint32_t kv_tokens_per_iteration = variant->map_kv_tokens_per_iteration;
    const uint32_t max_q_tokens = variant->map_max_q_tokens;
    KHM_REQUIRE(kv_tokens_per_iteration > 0, "BiDiBlockGQA KV-token iteration size must be positive");
    KHM_REQUIRE(max_q_tokens > 0, "BiDiBlockGQA Q-token range must contain tokens");

    for (uint32_t request = 0; request < num_requests; ++request)
        for (uint32_t offset = 0; offset < block_size; ++offset) req_slots_by_token[(uint64_t)request * block_size + offset] = req_slots[request];
    for (uint64_t t = 0; t < num_tokens; ++t) {
        flat_token_indices[t] = flat_query_token_indices[t];
        visible_kv_token_ranges[2 * t] = history_token_begins[t];
        visible_kv_token_ranges[2 * t + 1] = history_token_ends[t];
    }

    // build_metal_metadata (metadata.rs:182-337): request-local Q ranges of at most max_q_tokens rows
    std::vector<std::pair<uint64_t, uint64_t>> ranges;
    for (uint32_t request = 0; request < num_requests; ++request) {
        const uint64_t request_begin = (uint64_t)request * block_size, request_end = request_begin + block_size;
        for (uint64_t begin = request_begin; begin < request_end;) {
            const uint64_t end = std::min(begin + max_q_tokens, request_end);
            ranges.emplace_back(begin, end);
            begin = end;
        }
    }
    KHM_REQUIRE((uint64_t)max_sdpa_map_task_templates >= ranges.size() * 2, "BiDiBlockGQA TaskTemplate capacity holds %u, needs %llu",
                max_sdpa_map_task_templates, (unsigned long long)(ranges.size() * 2));
    KHM_REQUIRE((max_sdpa_map_task_templates & (max_sdpa_map_task_templates - 1)) == 0, "BiDiBlockGQA TaskTemplate capacity must be a power of two");
    // each range walks the union of its rows' history ranges; the per-row ranges stay the masks
    std::vector<std::pair<uint32_t, uint32_t>> history(ranges.size());
    std::vector<uint64_t> iterations(ranges.size());
    for (size_t r = 0; r < ranges.size(); ++r) {
        uint32_t begin = 0xffffffffu, end = 0;
        for (uint64_t t = ranges[r].first; t < ranges[r].second; ++t) {
            begin = std::min(begin, history_token_begins[t]);
            end = std::max(end, history_token_ends[t]);
        }
        history[r] = {begin, end};
        iterations[r] = ((uint64_t)(end - begin) + kv_tokens_per_iteration - 1) / kv_tokens_per_iteration;
        KHM_REQUIRE(iterations[r] <= (0xffffffffull - begin) / kv_tokens_per_iteration, "BiDiBlockGQA padded history-token range must fit u32");
    }
    const std::vector<uint64_t> splits = allocate_history_kv_splits(iterations, (uint64_t)max_sdpa_map_task_templates - ranges.size());

    uint64_t num_templates = 0;
    cu_sdpa_partial_outputs[0] = 0;
    for (size_t r = 0; r < ranges.size(); ++r) {
        q_token_ranges[2 * r] = (uint32_t)ranges[r].first;
        q_token_ranges[2 * r + 1] = (uint32_t)ranges[r].second;
        for (uint64_t split = 0; split < splits[r]; ++split) {
            const uint64_t iteration_begin = iterations[r] * split / splits[r];
            const uint64_t iteration_end = iterations[r] * (split + 1) / splits[r];
            KHM_REQUIRE(num_templates < max_sdpa_map_task_templates, "BiDiBlockGQA replay TaskTemplate count exceeds capacity");
            uint32_t* task = sdpa_map_task_templates + 3 * num_templates++;
            task[0] = (uint32_t)r;
            task[1] = history[r].first + (uint32_t)iteration_begin * kv_tokens_per_iteration;
            task[2] = std::min(history[r].second, history[r].first + (uint32_t)iteration_end * kv_tokens_per_iteration);
        }
        // the slot of the dense block partial: no Map task writes it
        KHM_REQUIRE(num_templates < max_sdpa_map_task_templates, "BiDiBlockGQA replay TaskTemplate count exceeds capacity");
        uint32_t* placeholder = sdpa_map_task_templates + 3 * num_templates++;
        placeholder[0] = placeholder[1] = placeholder[2] = 0xffffffffu;
        cu_sdpa_partial_outputs[r + 1] = (uint32_t)num_templates;
    }
    uint64_t num_total_templates = 0;
    KHM_REQUIRE(next_power_of_two_u64(num_templates, &num_total_templates) && num_total_templates <= max_sdpa_map_task_templates,
                "BiDiBlockGQA replay TaskTemplate count exceeds capacity");
    for (uint64_t i = num_templates * 3; i < num_total_templates * 3; ++i) sdpa_map_task_templates[i] = 0xffffffffu;

    // replay shape of the active prefix (metadata.rs:128-141)
    const uint64_t ranges_per_request = ((uint64_t)block_size + max_q_tokens - 1) / max_q_tokens;
    const uint64_t active_ranges = (uint64_t)num_active_requests * ranges_per_request;
    out_shape->num_tokens = num_active_requests * block_size;
    out_shape->num_total_tokens = (uint32_t)num_tokens;
    out_shape->num_q_token_tiles = (uint32_t)active_ranges;
    out_shape->num_total_q_token_tiles = (uint32_t)ranges.size();
    out_shape->num_sdpa_map_task_templates = cu_sdpa_partial_outputs[active_ranges];
    out_shape->num_total_sdpa_map_task_templates = (uint32_t)num_total_templates;
    out_shape->reduce_sdpa_partial_outputs = 1;
    return KHM_OK;
}
