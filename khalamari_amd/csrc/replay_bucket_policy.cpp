#include "replay_bucket_policy.h"

#include <algorithm>

#include "common.h"

namespace khm {

ReplayBucketPolicy::ReplayBucketPolicy(uint32_t max_capacity, const uint32_t* topology_boundaries, uint32_t num_boundaries)
    : max_capacity_(max_capacity) {
    static const uint32_t kBase[] = {1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 56, 64};
    for (uint32_t bucket : kBase) {
        if (bucket > max_capacity) break;
        buckets_.push_back(bucket);
    }
    // Above 64: lower + k * lower / 4 for k = 1..4, doubling lower, stopping before max_capacity.
    bool done = false;
    for (uint64_t lower = 64; !done && lower < max_capacity; lower *= 2) {
        const uint64_t step = lower / 4;
        for (uint64_t part = 1; part <= 4; ++part) {
            const uint64_t candidate = lower + step * part;
            if (candidate >= max_capacity) {
                done = true;
                break;
            }
            buckets_.push_back((uint32_t)candidate);
        }
    }
    for (uint32_t i = 0; i < num_boundaries; ++i) {
        const uint32_t boundary = topology_boundaries[i];
        if (boundary > 1 && boundary <= max_capacity) buckets_.push_back(boundary - 1);
    }
    buckets_.push_back(max_capacity);
    std::sort(buckets_.begin(), buckets_.end());
    buckets_.erase(std::unique(buckets_.begin(), buckets_.end()), buckets_.end());
}

uint32_t ReplayBucketPolicy::capacity(uint32_t active) const {
    return *std::lower_bound(buckets_.begin(), buckets_.end(), active);
}

}  // namespace khm

using namespace khm;

struct khm_replay_bucket_policy {
    ReplayBucketPolicy policy;
};

extern "C" int khm_replay_bucket_policy_create(uint32_t max_capacity, const uint32_t* topology_boundaries, uint32_t num_boundaries,
                                               khm_replay_bucket_policy** out) {
    clear_error();
    KHM_REQUIRE(out != nullptr, "policy output must not be null");
    KHM_REQUIRE(max_capacity > 0, "replay bucket capacity must be positive");
    for (uint32_t i = 0; i < num_boundaries; ++i) KHM_REQUIRE(topology_boundaries[i] > 0, "replay topology boundary must be positive");
    *out = new khm_replay_bucket_policy{ReplayBucketPolicy(max_capacity, topology_boundaries, num_boundaries)};
    return KHM_OK;
}

extern "C" void khm_replay_bucket_policy_destroy(khm_replay_bucket_policy* policy) { delete policy; }

extern "C" uint32_t khm_replay_bucket_policy_max_capacity(const khm_replay_bucket_policy* policy) { return policy->policy.max_capacity(); }

extern "C" int khm_replay_bucket_policy_buckets(const khm_replay_bucket_policy* policy, uint32_t* buckets, uint32_t capacity, uint32_t* count) {
    clear_error();
    KHM_REQUIRE(policy != nullptr && count != nullptr, "policy and count must not be null");
    const std::vector<uint32_t>& list = policy->policy.buckets();
    *count = (uint32_t)list.size();
    if (buckets != nullptr) {
        const size_t n = std::min<size_t>(capacity, list.size());
        std::copy(list.begin(), list.begin() + n, buckets);
    }
    return KHM_OK;
}

extern "C" int khm_replay_bucket_policy_capacity(const khm_replay_bucket_policy* policy, uint32_t active, uint32_t* out) {
    clear_error();
    KHM_REQUIRE(policy != nullptr && out != nullptr, "policy and out must not be null");
    KHM_REQUIRE(active > 0, "replay bucket requires active work");
    KHM_REQUIRE(active <= policy->policy.max_capacity(), "replay active work exceeds capacity");
    *out = policy->policy.capacity(active);
    return KHM_OK;
}

extern "C" int khm_replay_bucket_policy_capacity_allow_zero(const khm_replay_bucket_policy* policy, uint32_t active, uint32_t* out) {
    if (active == 0) {
        clear_error();
        KHM_REQUIRE(out != nullptr, "out must not be null");
        *out = 0;
        return KHM_OK;
    }
    return khm_replay_bucket_policy_capacity(policy, active, out);
}
