// Replay bucket policy: pads an active count up to the next recorded capacity.
// Behaviour of ReplayBucketPolicy (crates/inference-executor-core/src/replay.rs:1-87) and of
// GQAReplayBucketPolicy (crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:69-96).
#pragma once
#include <stdint.h>

#include <vector>

namespace khm {

class ReplayBucketPolicy {
public:
    // Base ladder 1,2,4,6,8,12,...,64, then four equal steps per octave, plus `boundary - 1` for every
    // topology boundary in (1, max], plus max itself; strictly increasing.
    ReplayBucketPolicy(uint32_t max_capacity, const uint32_t* topology_boundaries, uint32_t num_boundaries);
    explicit ReplayBucketPolicy(uint32_t max_capacity) : ReplayBucketPolicy(max_capacity, nullptr, 0) {}

    uint32_t max_capacity() const { return max_capacity_; }
    const std::vector<uint32_t>& buckets() const { return buckets_; }
    // First bucket >= active; requires 1 <= active <= max_capacity.
    uint32_t capacity(uint32_t active) const;

private:
    uint32_t max_capacity_;
    std::vector<uint32_t> buckets_;
};

struct GqaReplayBucketPolicy {
    ReplayBucketPolicy q_token_ranges;
    ReplayBucketPolicy map_task_templates;
    GqaReplayBucketPolicy(uint32_t max_tokens, uint32_t max_map_task_templates)
        : q_token_ranges(max_tokens), map_task_templates(max_map_task_templates) {}
};

}  // namespace khm
