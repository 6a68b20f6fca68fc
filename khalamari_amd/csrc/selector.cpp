// Work partitioner for the GQA SDPA component: Q-token ranges, KV splits, map task templates,
// cumulative partial counts and the padded replay shape.
//
// Behaviour follows crates/inference-executor-metal/src/attn/gqa/sdpa.rs:
//   RequestShape::from_batch (:21-41), Selector::{new, for_partitions} (:137-208),
//   select / select_partitioned / validate_* (:278-466), materialize_candidate (:476-664),
//   build_q_token_ranges (:780-819), allocate_kv_splits (:821-850), prefer_d256_page16_sliced_q (:852-869).
// The registry-comparison route of `select` is kept as is (it is deterministic integer logic with
// exact test vectors).  The lookup route (`for_lookup`, reference :210-272,667-778) is a table fitted
// to an Apple M3 Max; here it is replaced by a policy derived for 256 compute units, see lookup_route.
#include <algorithm>
#include <queue>
#include <vector>

#include "common.h"
#include "replay_bucket_policy.h"

namespace khm {

struct RangeWork {
    khm_q_token_range range;
    uint32_t num_kv_iterations;
    uint32_t num_kv_splits;
};

}  // namespace khm

using namespace khm;

struct khm_selector {
    khm_sdpa_config config;
    std::vector<khm_sdpa_variant> variants;
    khm_selector_limits limits;
    bool lookup = false;
};

struct khm_selection {
    khm_sdpa_variant variant;
    std::vector<khm_q_token_range> q_token_ranges;
    std::vector<khm_map_task_template> map_task_templates;
    std::vector<uint32_t> cu_partial_outputs;
    khm_gqa_replay_shape replay_shape;
    khm_selection_metrics metrics;
};

namespace khm {

static bool same_variant(const khm_sdpa_variant& a, const khm_sdpa_variant& b) {
    return a.map_kind == b.map_kind && a.map_max_q_tokens == b.map_max_q_tokens && a.map_max_q_heads == b.map_max_q_heads &&
           a.map_kv_tokens_per_iteration == b.map_kv_tokens_per_iteration && a.map_required_threads == b.map_required_threads &&
           a.kv_cache_tokens_per_page == b.kv_cache_tokens_per_page && a.reduce_max_q_tokens == b.reduce_max_q_tokens &&
           a.reduce_max_q_heads == b.reduce_max_q_heads && a.reduce_required_threads == b.reduce_required_threads;
}

static uint32_t ratio_of(const khm_sdpa_config& c) { return c.num_q_heads / c.num_kv_heads; }

// GQAReplayShape::validate (batch_metadata.rs:53-60).
static int validate_replay_shape(const khm_gqa_replay_shape& s) {
    KHM_REQUIRE(s.num_tokens > 0, "GQA replay shape requires tokens");
    KHM_REQUIRE(s.num_tokens <= s.num_total_tokens, "GQA replay tokens exceed the recorded capacity");
    KHM_REQUIRE(s.num_q_token_tiles > 0 && s.num_q_token_tiles <= s.num_tokens, "GQA replay Q-token tiles must be in 1..=tokens");
    KHM_REQUIRE(s.num_q_token_tiles <= s.num_total_q_token_tiles, "GQA replay Q-token tiles exceed the recorded capacity");
    KHM_REQUIRE(s.num_sdpa_map_task_templates >= s.num_q_token_tiles, "GQA replay needs a Map task template per Q-token tile");
    KHM_REQUIRE(s.num_sdpa_map_task_templates <= s.num_total_sdpa_map_task_templates,
                "GQA replay Map task templates exceed the recorded capacity");
    return KHM_OK;
}

static int build_q_token_ranges(const khm_request_shape* shapes, uint32_t num_requests, uint32_t max_q_tokens,
                                uint32_t kv_tokens_per_iteration, std::vector<RangeWork>* out) {
    uint64_t flat_request_begin = 0;
    for (uint32_t r = 0; r < num_requests; ++r) {
        const uint64_t flat_request_end = flat_request_begin + shapes[r].num_q_tokens;
        KHM_REQUIRE(flat_request_end <= 0xffffffffull, "GQA flat Q-token end must fit u32");
        uint64_t begin = flat_request_begin;
        while (begin < flat_request_end) {
            const uint64_t end = std::min<uint64_t>(begin + max_q_tokens, flat_request_end);
            const uint64_t visible = (uint64_t)shapes[r].num_history_tokens + (end - flat_request_begin);
            KHM_REQUIRE(visible <= 0xffffffffull, "GQA visible KV-token count must fit u32");
            const uint32_t iterations = div_ceil_u32((uint32_t)visible, kv_tokens_per_iteration);
            KHM_REQUIRE(iterations <= 0xffffffffu / kv_tokens_per_iteration, "GQA padded KV-token range must fit u32");
            RangeWork work;
            work.range = khm_q_token_range{r, (uint32_t)begin, (uint32_t)end, (uint32_t)visible};
            work.num_kv_iterations = iterations;
            work.num_kv_splits = 1;
            out->push_back(work);
            begin = end;
        }
        flat_request_begin = flat_request_end;
    }
    KHM_REQUIRE(!out->empty(), "GQA SDPA selector produced no Q-token ranges");
    return KHM_OK;
}

// Greedy: repeatedly give one more split to the range whose splits are currently the longest
// (ceil(iterations / splits)); ties go to the earlier range.  `min_iterations_per_split` > 1 (the lookup route only)
// keeps a range from being cut into splits shorter than that on average.
static void allocate_kv_splits(std::vector<RangeWork>& ranges, uint32_t max_map_task_templates, uint32_t min_iterations_per_split = 1) {
    const size_t count = ranges.size();
    if (count == max_map_task_templates) return;
    auto most_splits = [&](const RangeWork& range) { return std::max(range.num_kv_iterations / min_iterations_per_split, 1u); };
    if (count == 1) {
        ranges[0].num_kv_splits = std::min(most_splits(ranges[0]), max_map_task_templates);
        return;
    }
    struct Candidate {
        uint32_t work;
        size_t index;
        bool operator<(const Candidate& other) const {
            if (work != other.work) return work < other.work;
            return index > other.index;  // smaller index wins ties in a max-heap
        }
    };
    std::priority_queue<Candidate> heap;
    for (size_t i = 0; i < count; ++i) {
        if (ranges[i].num_kv_splits < most_splits(ranges[i]))
            heap.push(Candidate{div_ceil_u32(ranges[i].num_kv_iterations, ranges[i].num_kv_splits), i});
    }
    for (size_t used = count; used < max_map_task_templates; ++used) {
        if (heap.empty()) break;
        const Candidate top = heap.top();
        heap.pop();
        RangeWork& range = ranges[top.index];
        range.num_kv_splits += 1;
        if (range.num_kv_splits < most_splits(range))
            heap.push(Candidate{div_ceil_u32(range.num_kv_iterations, range.num_kv_splits), top.index});
    }
}

static bool mul_u64(uint64_t a, uint64_t b, uint64_t* out) { return !__builtin_mul_overflow(a, b, out); }

static int materialize_candidate(const khm_selector& selector, const khm_sdpa_variant& variant, const khm_request_shape* shapes,
                                 uint32_t num_requests, const GqaReplayBucketPolicy& policy, uint32_t num_total_tokens,
                                 bool has_slice, uint32_t kv_slice, bool direct_output, khm_selection* selection,
                                 uint32_t split_budget = 0, uint32_t min_iterations_per_split = 1) {
    const khm_selector_limits& limits = selector.limits;
    const uint32_t max_q_tokens = variant.map_max_q_tokens;
    const uint32_t stage = variant.map_kv_tokens_per_iteration;
    std::vector<RangeWork> ranges;
    if (int status = build_q_token_ranges(shapes, num_requests, max_q_tokens, stage, &ranges)) return status;
    if (has_slice) {
        uint64_t total = 0;
        for (RangeWork& work : ranges) {
            work.num_kv_splits = div_ceil_u32(work.range.num_visible_kv_tokens, kv_slice);
            total += work.num_kv_splits;
        }
        KHM_REQUIRE(total <= limits.max_map_task_templates, "GQA fixed slices exceed the Map task-template capacity");
    } else {
        uint32_t budget = limits.max_map_task_templates;
        if (split_budget != 0)
            budget = std::min(std::max<uint32_t>(split_budget, (uint32_t)ranges.size()), limits.max_map_task_templates);
        else if (variant.map_kind != KHM_MAP_SLICED_KV && stage == 32)
            budget = (uint32_t)std::min<uint64_t>((uint64_t)ranges.size() * 2, limits.max_map_task_templates);
        allocate_kv_splits(ranges, budget, min_iterations_per_split);
    }

    selection->variant = variant;
    selection->q_token_ranges.clear();
    selection->map_task_templates.clear();
    selection->cu_partial_outputs.assign(1, 0);
    uint32_t max_kv_iterations_per_split = 0;
    for (size_t index = 0; index < ranges.size(); ++index) {
        const RangeWork& work = ranges[index];
        selection->q_token_ranges.push_back(work.range);
        for (uint32_t split = 0; split < work.num_kv_splits; ++split) {
            uint32_t begin, end;
            if (has_slice) {
                const uint64_t b = (uint64_t)split * kv_slice;
                begin = (uint32_t)b;
                end = (uint32_t)std::min<uint64_t>(b + kv_slice, work.range.num_visible_kv_tokens);
            } else {
                const uint64_t iteration_begin = (uint64_t)work.num_kv_iterations * split / work.num_kv_splits;
                const uint64_t iteration_end = (uint64_t)work.num_kv_iterations * (split + 1) / work.num_kv_splits;
                begin = (uint32_t)iteration_begin * stage;
                end = std::min(work.range.num_visible_kv_tokens, (uint32_t)iteration_end * stage);
            }
            max_kv_iterations_per_split = std::max(max_kv_iterations_per_split, div_ceil_u32(end - begin, stage));
            selection->map_task_templates.push_back(khm_map_task_template{(uint32_t)index, begin, end});
        }
        KHM_REQUIRE(selection->map_task_templates.size() <= 0xffffffffull, "GQA SDPA partial-output count must fit u32");
        selection->cu_partial_outputs.push_back((uint32_t)selection->map_task_templates.size());
    }

    const uint32_t num_ranges = (uint32_t)selection->q_token_ranges.size();
    const uint32_t num_maps = (uint32_t)selection->map_task_templates.size();
    KHM_REQUIRE(num_maps <= limits.max_map_task_templates, "GQA SDPA Map task templates exceed the selector capacity");
    uint32_t num_tokens = 0;
    for (uint32_t r = 0; r < num_requests; ++r) num_tokens += shapes[r].num_q_tokens;
    KHM_REQUIRE(num_ranges <= policy.q_token_ranges.max_capacity(), "replay active work exceeds capacity");
    KHM_REQUIRE(num_maps > 0 && num_maps <= policy.map_task_templates.max_capacity(), "replay active work exceeds capacity");
    uint32_t total_ranges = policy.q_token_ranges.capacity(num_ranges);
    uint32_t total_maps = policy.map_task_templates.capacity(num_maps);
    if (direct_output) {
        // One direct Map owns each Q range: both padded domains share one extent.
        total_maps = total_ranges;
        KHM_REQUIRE(total_maps <= limits.max_map_task_templates, "GQA direct output exceeds the Map task-template capacity");
    }
    khm_gqa_replay_shape shape{};
    shape.num_tokens = num_tokens;
    shape.num_total_tokens = num_total_tokens;
    shape.num_q_token_tiles = num_ranges;
    shape.num_total_q_token_tiles = total_ranges;
    shape.num_sdpa_map_task_templates = num_maps;
    shape.num_total_sdpa_map_task_templates = total_maps;
    shape.reduce_sdpa_partial_outputs = !direct_output && (variant.map_kind != KHM_MAP_SLICED_KV || num_maps > num_tokens);
    if (int status = validate_replay_shape(shape)) return status;
    selection->replay_shape = shape;

    khm_selection_metrics metrics{};
    if (!direct_output) {
        for (const RangeWork& work : ranges)
            metrics.num_active_partial_state_groups +=
                (uint64_t)(work.range.flat_q_token_end - work.range.flat_q_token_begin) * work.num_kv_splits;
        metrics.num_reserved_partial_state_groups = (uint64_t)num_maps * max_q_tokens;
        metrics.num_replay_reserved_partial_state_groups = (uint64_t)total_maps * max_q_tokens;
    }
    KHM_REQUIRE(metrics.num_replay_reserved_partial_state_groups <= limits.partial_state_group_capacity,
                "GQA SDPA replay exceeds its partial-state-group capacity");
    for (const khm_map_task_template& t : selection->map_task_templates) {
        const khm_q_token_range& range = selection->q_token_ranges[t.q_token_range_index];
        const uint64_t staged = (uint64_t)div_ceil_u32(t.kv_token_end - t.kv_token_begin, stage) * stage;
        metrics.num_scheduled_qk_token_pairs += staged * max_q_tokens;
        metrics.num_active_qk_token_pairs += staged * (range.flat_q_token_end - range.flat_q_token_begin);
    }
    const uint32_t head_ranges = div_ceil_u32(ratio_of(selector.config), variant.map_max_q_heads);
    metrics.num_map_threadblocks_per_kv_head = (uint64_t)num_maps * head_ranges;
    metrics.num_map_simdgroup_waves_per_kv_head = metrics.num_map_threadblocks_per_kv_head * (variant.map_required_threads / 32);
    for (uint32_t r = 0; r < num_requests; ++r) {
        const uint64_t q = shapes[r].num_q_tokens;
        uint64_t pairs, causal;
        KHM_REQUIRE(mul_u64(q, (uint64_t)shapes[r].num_history_tokens + 1, &pairs) && mul_u64(q, q > 0 ? q - 1 : 0, &causal) &&
                        !__builtin_add_overflow(pairs, causal / 2, &pairs) &&
                        !__builtin_add_overflow(metrics.num_logical_qk_token_pairs, pairs, &metrics.num_logical_qk_token_pairs),
                    "GQA logical query-key pair count must fit u64");
    }
    KHM_REQUIRE(mul_u64(metrics.num_active_partial_state_groups, selector.config.num_q_heads, &metrics.num_active_partial_states),
                "GQA active partial-state count must fit u64");
    metrics.max_kv_iterations_per_split = max_kv_iterations_per_split;
    selection->metrics = metrics;
    return KHM_OK;
}

static uint64_t selection_overhead_score(const khm_selection_metrics& m) {
    return m.num_map_threadblocks_per_kv_head + m.num_map_simdgroup_waves_per_kv_head + m.num_active_partial_state_groups +
           m.num_replay_reserved_partial_state_groups;
}

static bool prefer_d256_page16_sliced_q(const khm_selection& sliced_kv, const khm_selection& sliced_q) {
    const uint64_t score = sliced_kv.metrics.num_logical_qk_token_pairs +
                           std::min(selection_overhead_score(sliced_kv.metrics), selection_overhead_score(sliced_q.metrics));
    uint64_t doubled;
    const bool utilised = mul_u64(sliced_q.metrics.num_active_qk_token_pairs, 2, &doubled) &&
                          doubled >= sliced_q.metrics.num_scheduled_qk_token_pairs;
    return utilised && score >= 2048;
}

static int validate_request_shapes(const khm_selector& selector, const khm_request_shape* shapes, uint32_t num_requests,
                                   const GqaReplayBucketPolicy& policy, uint32_t num_total_tokens, uint32_t* num_tokens_out) {
    KHM_REQUIRE(policy.q_token_ranges.max_capacity() == selector.limits.max_tokens,
                "GQA replay bucket policy must match the SDPA token capacity");
    KHM_REQUIRE(policy.map_task_templates.max_capacity() == selector.limits.max_map_task_templates,
                "GQA replay bucket policy must match the SDPA Map task-template capacity");
    KHM_REQUIRE(num_requests > 0 && shapes != nullptr, "GQA SDPA selector requires requests");
    uint64_t num_tokens = 0;
    for (uint32_t r = 0; r < num_requests; ++r) {
        num_tokens += shapes[r].num_q_tokens;
        KHM_REQUIRE(num_tokens <= 0xffffffffull, "GQA SDPA token count must fit u32");
        KHM_REQUIRE((uint64_t)shapes[r].num_history_tokens + shapes[r].num_q_tokens <= 0xffffffffull,
                    "GQA request context length must fit u32");
    }
    KHM_REQUIRE(num_tokens > 0, "GQA SDPA selector requires Q tokens");
    KHM_REQUIRE(num_tokens <= selector.limits.max_tokens, "GQA SDPA tokens exceed the selector capacity");
    KHM_REQUIRE(num_tokens <= num_total_tokens, "GQA active token count must not exceed the total token count");
    KHM_REQUIRE(num_total_tokens <= policy.q_token_ranges.max_capacity(),
                "GQA total token count must not exceed the metadata capacity");
    *num_tokens_out = (uint32_t)num_tokens;
    return KHM_OK;
}

// ---------------------------------------------------------------------------------------------
// Lookup policy for MI355X: 256 compute units, each comfortable with 2-4 resident Map blocks.
//
//   * Q tile.  Per-request query capacity q = next_pow2(min(max q_len, 32)).
//       q == 1           -> SlicedKv with all of a KV head's Q heads in one block when ratio <= 8,
//                           otherwise a one-token sliced-Q tile that still reads K/V once per KV head.
//       q * ratio <= 64  -> one sliced-Q tile of q tokens x ratio heads (verify blocks).
//       q >= 16          -> dense prefill: the largest power-of-two token tile with tile * ratio <= 256 (192 at D 256).
//       otherwise        -> the largest power-of-two token tile with tile * ratio <= 64.
//   * KV splits.  A block streams its split once, so splits only need to be short enough to fill the
//     chip: kTargetBlocks blocks in total and not one more, because the verify kernels hold two (bf16 pages) or four
//     (FP8 pages) blocks per compute unit and blocks beyond a whole number of rounds run in a nearly empty one (1448 blocks
//     of a batch of 16 speculative requests took two rounds of 1024 slots on FP8 pages).  The template budget is handed
//     out greedily, one more split at a time to the range whose splits are currently the longest, so all blocks end up
//     about equally long, in whole 64-token iterations; a range is never cut into splits shorter than kMinSlice tokens on
//     average (shorter ones pay more in partial traffic than they gain in parallelism).
//     When the unsplit grid already has kTargetBlocks / 2 blocks, sliced-Q runs unsplit with direct output.
// ---------------------------------------------------------------------------------------------
constexpr uint64_t kTargetBlocks = 1024;
constexpr uint32_t kMinSlice = 256;
constexpr uint32_t kMaxColumns = 64;          // small-tile split-KV kernel (decode, verify)
constexpr uint32_t kMaxPrefillColumns = 256;  // LDS-shared K/V tile kernel (dense prefill chunks)

static int lookup_variant(const khm_sdpa_config& config, uint32_t queries, khm_sdpa_variant* out) {
    const uint32_t ratio = ratio_of(config);
    if (queries == 1 && ratio <= 8) {
        const uint32_t clamped = std::min(std::max(config.head_dim, 32u), 256u);
        return khm_sdpa_variant_sliced_kv(&config, next_power_of_two(clamped), 128, ratio, out);
    }
    // Chunks of 16+ tokens per request are compute-bound: give them the widest tile so each K/V byte staged in
    // LDS feeds as many MFMA columns as possible.  Narrower blocks are bandwidth-bound and stay on small tiles.
    // At D 256 the 256-column tile does not fit the register file (it spills): tiles stop at 192 columns (twelve waves of
    // one column tile: 32 tokens x 6 heads of a group-6 model) and otherwise at 128.
    const uint32_t prefill_columns = config.head_dim > 128 ? 3 * kMaxPrefillColumns / 4 : kMaxPrefillColumns;
    const uint32_t max_columns = queries >= 16 ? prefill_columns : kMaxColumns;
    uint32_t heads = std::min(ratio, max_columns);
    uint32_t tile = queries;
    while (tile > 1 && (uint64_t)tile * heads > max_columns) tile /= 2;
    return khm_sdpa_variant_sliced_q(&config, KHM_MAP_Q_TOKENS_AND_HEADS, tile, 64, heads, out);
}

// Outputs: `direct` (one unsplit Map per Q range, final output) or else `split_budget`, the number of Map task templates
// to hand out over the Q ranges.
static int lookup_route(const khm_selector& selector, const khm_request_shape* shapes, uint32_t num_requests,
                        khm_sdpa_variant* variant, uint32_t* slice, bool* direct, uint32_t* split_budget) {
    const khm_sdpa_config& config = selector.config;
    uint32_t max_q = 0, end = 0;
    for (uint32_t r = 0; r < num_requests; ++r) {
        max_q = std::max(max_q, shapes[r].num_q_tokens);
        end = std::max(end, shapes[r].num_history_tokens + shapes[r].num_q_tokens);
    }
    const uint32_t queries = next_power_of_two(std::min(max_q, 32u));
    if (int status = lookup_variant(config, queries, variant)) return status;
    const uint64_t tile = variant->map_max_q_tokens;
    const uint64_t blocks_per_map = (uint64_t)config.num_kv_heads * div_ceil_u32(ratio_of(config), variant->map_max_q_heads);
    uint64_t num_ranges = 0;
    for (uint32_t r = 0; r < num_requests; ++r) num_ranges += div_ceil_u64(shapes[r].num_q_tokens, tile);
    const bool can_direct = variant->map_kind != KHM_MAP_SLICED_KV;
    if (can_direct && (num_ranges * blocks_per_map >= kTargetBlocks / 2 || end <= kMinSlice)) {
        *slice = end;
        *direct = true;
        return KHM_OK;
    }
    // a whole number of blocks per template: round the budget down so that the grid does not exceed kTargetBlocks
    const uint64_t wanted_maps = std::max<uint64_t>(kTargetBlocks / blocks_per_map, num_ranges);
    KHM_REQUIRE(selector.limits.max_map_task_templates >= num_ranges, "GQA Q-token ranges exceed the Map task-template capacity");
    *slice = end;
    *direct = false;
    *split_budget = (uint32_t)std::min<uint64_t>(wanted_maps, selector.limits.max_map_task_templates);
    return KHM_OK;
}

static int select_impl(const khm_selector& selector, const khm_request_shape* shapes, uint32_t num_requests,
                       const GqaReplayBucketPolicy& policy, uint32_t num_total_tokens, khm_selection* result) {
    uint32_t num_tokens = 0;
    if (int status = validate_request_shapes(selector, shapes, num_requests, policy, num_total_tokens, &num_tokens)) return status;
    const khm_sdpa_config& config = selector.config;
    if (selector.lookup) {
        khm_sdpa_variant variant;
        uint32_t slice = 0, split_budget = 0;
        bool direct = false;
        if (int status = lookup_route(selector, shapes, num_requests, &variant, &slice, &direct, &split_budget)) return status;
        if (direct)
            return materialize_candidate(selector, variant, shapes, num_requests, policy, num_total_tokens, true, slice, true, result);
        const uint32_t min_iterations = std::max(kMinSlice / variant.map_kv_tokens_per_iteration, 1u);
        if (int status = materialize_candidate(selector, variant, shapes, num_requests, policy, num_total_tokens, false, 0, false,
                                               result, split_budget, min_iterations))
            return status;
        // nothing was split (short contexts): sliced-Q then writes its output directly, no Reduce
        if (variant.map_kind != KHM_MAP_SLICED_KV && result->map_task_templates.size() == result->q_token_ranges.size())
            return materialize_candidate(selector, variant, shapes, num_requests, policy, num_total_tokens, true, slice, true, result);
        return KHM_OK;
    }
    auto materialize = [&](const khm_sdpa_variant& variant, khm_selection* out) {
        return materialize_candidate(selector, variant, shapes, num_requests, policy, num_total_tokens, false, 0, false, out);
    };
    const khm_sdpa_variant* sliced_kv = nullptr;
    std::vector<const khm_sdpa_variant*> sliced_q;
    for (const khm_sdpa_variant& v : selector.variants) {
        if (v.map_kind == KHM_MAP_SLICED_KV) {
            if (!sliced_kv) sliced_kv = &v;
        } else {
            sliced_q.push_back(&v);
        }
    }
    if (sliced_q.empty()) {
        KHM_REQUIRE(sliced_kv != nullptr, "GQA SDPA registry requires an execution");
        return materialize(*sliced_kv, result);
    }
    const khm_sdpa_variant& first_sliced_q = *sliced_q.front();
    if (sliced_kv == nullptr) return materialize(first_sliced_q, result);

    // Q-range density rejects sliced-Q before any KV split allocation.
    uint64_t num_ranges = 0;
    for (uint32_t r = 0; r < num_requests; ++r) num_ranges += div_ceil_u32(shapes[r].num_q_tokens, first_sliced_q.map_max_q_tokens);
    if ((uint64_t)num_tokens < 2 * num_ranges) return materialize(*sliced_kv, result);

    uint32_t full_q_heads = first_sliced_q.map_max_q_heads;
    for (size_t i = 1; i < sliced_q.size(); ++i) full_q_heads = std::max(full_q_heads, sliced_q[i]->map_max_q_heads);
    const bool d128_profile = config.head_dim == 128 && (config.tokens_per_page == 8 || config.tokens_per_page == 16);
    uint32_t desired_q_heads = full_q_heads;
    if (!d128_profile && (uint64_t)num_tokens < 4 * num_ranges) desired_q_heads = std::min(div_ceil_u32(ratio_of(config), 2), full_q_heads);
    const uint32_t desired_kv_tokens = (config.head_dim == 256 && num_tokens >= 1024 && (uint64_t)num_tokens >= 4 * num_ranges) ? 32 : 16;
    // max_by_key(stage == desired): the last maximal element wins, as Iterator::max_by_key does.
    const khm_sdpa_variant* chosen = nullptr;
    bool chosen_key = false;
    for (const khm_sdpa_variant* v : sliced_q) {
        if (v->map_max_q_heads != desired_q_heads) continue;
        const bool key = v->map_kv_tokens_per_iteration == desired_kv_tokens;
        if (chosen == nullptr || key >= chosen_key) {
            chosen = v;
            chosen_key = key;
        }
    }
    if (chosen == nullptr) chosen = &first_sliced_q;
    khm_selection q_selection;
    if (int status = materialize(*chosen, &q_selection)) return status;
    if (config.head_dim == 256 && config.tokens_per_page == 16) {
        khm_selection kv_selection;
        if (int status = materialize(*sliced_kv, &kv_selection)) return status;
        if (!prefer_d256_page16_sliced_q(kv_selection, q_selection)) {
            *result = std::move(kv_selection);
            return KHM_OK;
        }
    }
    *result = std::move(q_selection);
    return KHM_OK;
}

static int make_selector(const khm_sdpa_config* config, const khm_sdpa_variant* variants, uint32_t num_variants, uint64_t max_tokens,
                         uint64_t max_maps, uint64_t partial_capacity, khm_selector** out) {
    if (int status = validate_sdpa_config(config)) return status;
    KHM_REQUIRE(out != nullptr, "selector output must not be null");
    KHM_REQUIRE(variants != nullptr && num_variants > 0, "GQA SDPA registry requires an execution variant");
    for (uint32_t i = 0; i < num_variants; ++i)
        KHM_REQUIRE(variant_supports(variants[i], *config), "GQA SDPA registry contains an unsupported execution variant");
    KHM_REQUIRE(max_tokens > 0, "GQA SDPA selector requires tokens");
    KHM_REQUIRE(max_maps > 0, "GQA SDPA selector requires Map task templates");
    KHM_REQUIRE(partial_capacity > 0, "GQA SDPA selector requires partial-state groups");
    KHM_REQUIRE(max_tokens <= 0xffffffffull, "GQA SDPA token capacity must fit u32");
    KHM_REQUIRE(max_maps <= 0xffffffffull, "GQA SDPA Map task-template capacity must fit u32");
    auto* selector = new khm_selector();
    selector->config = *config;
    selector->variants.assign(variants, variants + num_variants);
    selector->limits = khm_selector_limits{(uint32_t)max_tokens, (uint32_t)max_maps, partial_capacity};
    *out = selector;
    return KHM_OK;
}

}  // namespace khm

extern "C" int khm_request_shapes_from_batch(const uint32_t* token_indices, const uint32_t* cu_tokens, uint32_t num_requests,
                                             khm_request_shape* out) {
    clear_error();
    KHM_REQUIRE(token_indices != nullptr && cu_tokens != nullptr && out != nullptr, "batch arrays must not be null");
    KHM_REQUIRE(cu_tokens[0] == 0, "GQA batch cu_tokens must start at zero");
    for (uint32_t r = 0; r < num_requests; ++r) {
        KHM_REQUIRE(cu_tokens[r] <= cu_tokens[r + 1], "GQA batch cu_tokens must be nondecreasing");
        const uint32_t q = cu_tokens[r + 1] - cu_tokens[r];
        KHM_REQUIRE(q > 0, "GQA requests must contain Q tokens");
        KHM_REQUIRE((uint64_t)token_indices[r] + q <= 0xffffffffull, "GQA request context length must fit u32");
        out[r] = khm_request_shape{token_indices[r], q};
    }
    return KHM_OK;
}

extern "C" int khm_selector_create(const khm_sdpa_config* config, const khm_sdpa_variant* variants, uint32_t num_variants,
                                   uint64_t max_tokens, uint64_t max_map_task_templates, uint64_t partial_state_group_capacity,
                                   khm_selector** out) {
    clear_error();
    return make_selector(config, variants, num_variants, max_tokens, max_map_task_templates, partial_state_group_capacity, out);
}

extern "C" int khm_selector_create_for_partitions(const khm_sdpa_config* config, const khm_sdpa_variant* variants,
                                                  const uint32_t* max_kv_splits, uint32_t num_variants, uint32_t max_tokens,
                                                  uint32_t max_requests, khm_selector** out) {
    clear_error();
    KHM_REQUIRE(max_tokens > 0, "GQA partition envelope requires tokens");
    KHM_REQUIRE(max_requests > 0, "GQA partition envelope requires requests");
    KHM_REQUIRE(variants != nullptr && max_kv_splits != nullptr && num_variants > 0, "GQA SDPA registry requires an execution variant");
    max_requests = std::min(max_requests, max_tokens);
    std::vector<uint32_t> maps(num_variants);
    uint32_t max_maps = 0;
    for (uint32_t i = 0; i < num_variants; ++i) {
        KHM_REQUIRE(variants[i].map_max_q_tokens > 0, "GQA SDPA registry contains an unsupported execution variant");
        const uint32_t max_ranges = max_requests + (max_tokens - max_requests) / variants[i].map_max_q_tokens;
        KHM_REQUIRE(max_kv_splits[i] > 0, "GQA partition envelope requires KV splits");
        const uint64_t product = (uint64_t)max_ranges * max_kv_splits[i];
        KHM_REQUIRE(product <= 0xffffffffull, "GQA partition Map task-template count must fit u32");
        maps[i] = (uint32_t)product;
        max_maps = std::max(max_maps, maps[i]);
    }
    const ReplayBucketPolicy buckets(max_maps);
    uint64_t partial_capacity = 0;
    for (uint32_t i = 0; i < num_variants; ++i)
        partial_capacity = std::max<uint64_t>(partial_capacity, (uint64_t)buckets.capacity(maps[i]) * variants[i].map_max_q_tokens);
    return make_selector(config, variants, num_variants, max_tokens, max_maps, partial_capacity, out);
}

extern "C" int khm_selector_create_for_lookup(const khm_sdpa_config* config, uint64_t max_tokens, const khm_page_table_layout* layout,
                                              khm_selector** out) {
    clear_error();
    if (int status = validate_sdpa_config(config)) return status;
    KHM_REQUIRE(layout != nullptr && layout->num_req_slots > 0 && layout->num_blocks > 0 && layout->num_gqa_layers > 0 &&
                    layout->num_page_ids_per_block > 0,
                "GQA page-table layout must be positive");
    KHM_REQUIRE(max_tokens > 0 && max_tokens <= 0xffffffffull, "GQA lookup requires tokens");
    std::string why;
    khm_sdpa_variant probe;
    const bool built = khm_sdpa_variant_sliced_kv(config, 128, 128, 1, &probe) == KHM_OK &&
                       kernel_family(*config, probe, KHM_DTYPE_BF16, &why) != 0;
    clear_error();
    if (!built) {
        // Geometries without a gfx950 kernel keep the registry route and its worst-case envelope (sdpa.rs:216-228).
        khm_sdpa_variant variants[8];
        uint32_t count = 0;
        if (int status = khm_sdpa_registry_new(config, variants, 8, &count)) return status;
        uint32_t max_tile = 1;
        for (uint32_t i = 0; i < count; ++i) max_tile = std::max(max_tile, variants[i].map_max_q_tokens);
        return make_selector(config, variants, count, max_tokens, max_tokens, max_tokens * max_tile, out);
    }
    const uint64_t pages = (uint64_t)layout->num_blocks * layout->num_page_ids_per_block;
    const uint64_t max_visible = pages * config->tokens_per_page;
    KHM_REQUIRE(max_visible <= 0xffffffffull, "GQA page-table token capacity must fit u32");
    std::vector<khm_sdpa_variant> variants;
    for (uint32_t queries = 1; queries <= 32; queries *= 2) {
        if (queries > next_power_of_two((uint32_t)std::min<uint64_t>(max_tokens, 32))) break;
        khm_sdpa_variant v;
        if (int status = lookup_variant(*config, queries, &v)) return status;
        bool seen = false;
        for (const khm_sdpa_variant& existing : variants) seen = seen || same_variant(existing, v);
        if (!seen) variants.push_back(v);
    }
    // Slices are never shorter than kMinSlice unless capacity forces them longer, so a request needs at
    // most ceil(max_visible / kMinSlice) splits per range, and the chip-filling target adds kTargetBlocks.
    const uint64_t max_splits = div_ceil_u64(max_visible, kMinSlice);
    uint64_t max_maps = std::max<uint64_t>(max_tokens, (uint64_t)layout->num_req_slots * max_splits + kTargetBlocks);
    max_maps = std::max<uint64_t>(max_maps, max_tokens + kTargetBlocks);
    KHM_REQUIRE(max_maps <= 0xffffffffull, "GQA Map task-template capacity must fit u32");
    uint32_t max_tile = 1;
    for (const khm_sdpa_variant& v : variants) max_tile = std::max(max_tile, v.map_max_q_tokens);
    if (int status = make_selector(config, variants.data(), (uint32_t)variants.size(), max_tokens, max_maps, max_maps * max_tile, out))
        return status;
    (*out)->lookup = true;
    return KHM_OK;
}

extern "C" void khm_selector_destroy(khm_selector* selector) { delete selector; }

extern "C" int khm_selector_limits_get(const khm_selector* selector, khm_selector_limits* out) {
    clear_error();
    KHM_REQUIRE(selector != nullptr && out != nullptr, "selector and out must not be null");
    *out = selector->limits;
    return KHM_OK;
}

extern "C" int khm_selector_variants(const khm_selector* selector, khm_sdpa_variant* variants, uint32_t capacity, uint32_t* count) {
    clear_error();
    KHM_REQUIRE(selector != nullptr && count != nullptr, "selector and count must not be null");
    *count = (uint32_t)selector->variants.size();
    if (variants != nullptr) {
        if (capacity < selector->variants.size()) return fail(KHM_ERR_CAPACITY, "selector holds %zu variants", selector->variants.size());
        std::copy(selector->variants.begin(), selector->variants.end(), variants);
    }
    return KHM_OK;
}

extern "C" int khm_selector_select(const khm_selector* selector, const khm_request_shape* request_shapes, uint32_t num_requests,
                                   uint32_t policy_max_tokens, uint32_t policy_max_map_task_templates, uint32_t num_total_tokens,
                                   khm_selection** out) {
    clear_error();
    KHM_REQUIRE(selector != nullptr && out != nullptr, "selector and out must not be null");
    KHM_REQUIRE(policy_max_tokens > 0 && policy_max_map_task_templates > 0, "replay bucket capacity must be positive");
    const GqaReplayBucketPolicy policy(policy_max_tokens, policy_max_map_task_templates);
    auto* selection = new khm_selection();
    const int status = select_impl(*selector, request_shapes, num_requests, policy, num_total_tokens, selection);
    if (status != KHM_OK) {
        delete selection;
        return status;
    }
    *out = selection;
    return KHM_OK;
}

extern "C" int khm_selector_select_partitioned(const khm_selector* selector, const khm_sdpa_variant* variant, uint32_t kv_slice,
                                               int direct_output, const khm_request_shape* request_shapes, uint32_t num_requests,
                                               uint32_t policy_max_tokens, uint32_t policy_max_map_task_templates,
                                               uint32_t num_total_tokens, khm_selection** out) {
    clear_error();
    KHM_REQUIRE(selector != nullptr && variant != nullptr && out != nullptr, "selector, variant and out must not be null");
    KHM_REQUIRE(policy_max_tokens > 0 && policy_max_map_task_templates > 0, "replay bucket capacity must be positive");
    const GqaReplayBucketPolicy policy(policy_max_tokens, policy_max_map_task_templates);
    uint32_t num_tokens = 0;
    if (int status = validate_request_shapes(*selector, request_shapes, num_requests, policy, num_total_tokens, &num_tokens)) return status;
    bool member = false;
    for (const khm_sdpa_variant& v : selector->variants) member = member || same_variant(v, *variant);
    KHM_REQUIRE(member, "GQA route must belong to its initialized registry");
    KHM_REQUIRE(kv_slice > 0, "GQA KV slice must contain tokens");
    if (direct_output) {
        uint32_t max_visible = 0;
        for (uint32_t r = 0; r < num_requests; ++r)
            max_visible = std::max(max_visible, request_shapes[r].num_history_tokens + request_shapes[r].num_q_tokens);
        KHM_REQUIRE(variant->map_kind != KHM_MAP_SLICED_KV, "GQA SlicedKv requires Map/Reduce output");
        KHM_REQUIRE(kv_slice >= max_visible, "GQA direct output requires an unsplit KV range");
    }
    auto* selection = new khm_selection();
    const int status = materialize_candidate(*selector, *variant, request_shapes, num_requests, policy, num_total_tokens, true, kv_slice,
                                             direct_output != 0, selection);
    if (status != KHM_OK) {
        delete selection;
        return status;
    }
    *out = selection;
    return KHM_OK;
}

extern "C" void khm_selection_destroy(khm_selection* selection) { delete selection; }

extern "C" int khm_selection_variant(const khm_selection* selection, khm_sdpa_variant* out) {
    clear_error();
    KHM_REQUIRE(selection != nullptr && out != nullptr, "selection and out must not be null");
    *out = selection->variant;
    return KHM_OK;
}

extern "C" int khm_selection_direct_output(const khm_selection* selection) {
    return selection->variant.map_kind != KHM_MAP_SLICED_KV && !selection->replay_shape.reduce_sdpa_partial_outputs ? 1 : 0;
}

extern "C" int khm_selection_replay_shape(const khm_selection* selection, khm_gqa_replay_shape* out) {
    clear_error();
    KHM_REQUIRE(selection != nullptr && out != nullptr, "selection and out must not be null");
    *out = selection->replay_shape;
    return KHM_OK;
}

extern "C" int khm_selection_metrics_get(const khm_selection* selection, khm_selection_metrics* out) {
    clear_error();
    KHM_REQUIRE(selection != nullptr && out != nullptr, "selection and out must not be null");
    *out = selection->metrics;
    return KHM_OK;
}

extern "C" uint32_t khm_selection_num_q_token_ranges(const khm_selection* selection) { return (uint32_t)selection->q_token_ranges.size(); }
extern "C" uint32_t khm_selection_num_map_task_templates(const khm_selection* selection) {
    return (uint32_t)selection->map_task_templates.size();
}

extern "C" int khm_selection_q_token_ranges(const khm_selection* selection, khm_q_token_range* out, uint32_t capacity) {
    clear_error();
    KHM_REQUIRE(selection != nullptr && out != nullptr, "selection and out must not be null");
    if (capacity < selection->q_token_ranges.size()) return fail(KHM_ERR_CAPACITY, "selection holds %zu Q-token ranges", selection->q_token_ranges.size());
    std::copy(selection->q_token_ranges.begin(), selection->q_token_ranges.end(), out);
    return KHM_OK;
}

extern "C" int khm_selection_map_task_templates(const khm_selection* selection, khm_map_task_template* out, uint32_t capacity) {
    clear_error();
    KHM_REQUIRE(selection != nullptr && out != nullptr, "selection and out must not be null");
    if (capacity < selection->map_task_templates.size())
        return fail(KHM_ERR_CAPACITY, "selection holds %zu Map task templates", selection->map_task_templates.size());
    std::copy(selection->map_task_templates.begin(), selection->map_task_templates.end(), out);
    return KHM_OK;
}

extern "C" int khm_selection_cu_partial_outputs(const khm_selection* selection, uint32_t* out, uint32_t capacity) {
    clear_error();
    KHM_REQUIRE(selection != nullptr && out != nullptr, "selection and out must not be null");
    if (capacity < selection->cu_partial_outputs.size())
        return fail(KHM_ERR_CAPACITY, "selection holds %zu cumulative partial counts", selection->cu_partial_outputs.size());
    std::copy(selection->cu_partial_outputs.begin(), selection->cu_partial_outputs.end(), out);
    return KHM_OK;
}
