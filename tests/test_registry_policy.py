"""Static capability registry and the replay bucket policy (host only)."""
import pytest

from khalamari_amd import sdpa
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, KhmError
from khalamari_amd.replay import ReplayBucketPolicy


def _config(head_dim, ratio, tpp, dtype=DTYPE_BF16):
    return sdpa.Config(dtype, 2 * ratio, 2, head_dim, tpp)


def test_registry_filters_static_execution_capabilities():
    # components/gqa/sdpa.rs:346-376
    counts = [(256, 6, 32, 4), (256, 6, 16, 4), (256, 6, 8, 4), (128, 8, 16, 2), (128, 8, 8, 2), (256, 8, 4, 1)]
    for head_dim, ratio, tpp, expected in counts:
        config = _config(head_dim, ratio, tpp)
        registry = sdpa.Registry(config)
        assert len(registry.variants()) == expected, (head_dim, ratio, tpp)
        assert all(sdpa.supports(v, config) for v in registry.variants())


def test_variant_constructors_follow_the_reference_geometry():
    config = _config(128, 8, 16)
    v = sdpa.ExecutionVariant.sliced_kv(config, 128, 128, 8)
    assert (v.map_kind, v.map_max_q_tokens, v.map_max_q_heads, v.reduce_max_q_tokens, v.reduce_max_q_heads, v.reduce_required_threads) == \
        (sdpa.MAP_SLICED_KV, 1, 8, 1, 2, 256)
    assert sdpa.ExecutionVariant.sliced_q(config, sdpa.MAP_Q_TOKENS_PER_HEAD, 16, 16, 8).map_required_threads == 2 * 8 * 32
    assert sdpa.ExecutionVariant.sliced_q(config, sdpa.MAP_Q_HEADS_PER_TOKEN, 4, 16, 8).map_required_threads == 1 * 4 * 32
    assert sdpa.ExecutionVariant.sliced_q(config, sdpa.MAP_Q_TOKENS_AND_HEADS, 4, 16, 6).map_required_threads == 3 * 32
    with pytest.raises(KhmError):
        sdpa.ExecutionVariant.sliced_q(config, sdpa.MAP_Q_TOKENS_PER_HEAD, 3, 16, 8)       # tile not in {1,..,32}
    with pytest.raises(KhmError):
        sdpa.ExecutionVariant.sliced_q(config, sdpa.MAP_Q_TOKENS_PER_HEAD, 8, 16, 9)       # more heads than the ratio
    with pytest.raises(KhmError):
        sdpa.ExecutionVariant.sliced_kv(config, 128, 96, 8)                                 # threads not a power of two
    with pytest.raises(KhmError):
        sdpa.ExecutionVariant.sliced_q(_config(192, 8, 8), sdpa.MAP_Q_TOKENS_PER_HEAD, 8, 16, 8)  # unsupported profile


def test_kernel_availability_is_reported_separately_from_legality():
    config = _config(128, 8, 16)
    assert sdpa.has_kernel(config, sdpa.ExecutionVariant.sliced_kv(config, 128, 128, 8))
    f32 = _config(128, 8, 16, DTYPE_F32)
    assert not sdpa.has_kernel(f32, sdpa.ExecutionVariant.sliced_kv(f32, 128, 128, 8))
    odd = _config(64, 4, 16)
    assert sdpa.supports(sdpa.ExecutionVariant.sliced_kv(odd, 64, 64, 4), odd)
    assert not sdpa.has_kernel(odd, sdpa.ExecutionVariant.sliced_kv(odd, 64, 64, 4))


# ---- crates/inference-executor-core/src/replay.rs:93-171 ------------------------------------------------------

def test_default_policy_extends_past_64_and_includes_terminal_capacity():
    assert ReplayBucketPolicy(128).buckets() == [1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 56, 64, 80, 96, 112, 128]
    assert ReplayBucketPolicy(70).buckets()[-1] == 70
    assert ReplayBucketPolicy(6).buckets() == [1, 2, 4, 6]


def test_buckets_remain_ordered_at_extension_boundaries_and_u32_limit():
    for max_capacity in [65, 79, 80, 81, 127, 128, 129, 0xFFFFFFFF]:
        policy = ReplayBucketPolicy(max_capacity)
        buckets = policy.buckets()
        assert buckets[-1] == max_capacity
        assert policy.capacity(max_capacity) == max_capacity
        assert all(a < b for a, b in zip(buckets, buckets[1:]))


def test_capacity_uses_the_first_bucket_that_contains_active_work():
    policy = ReplayBucketPolicy(64)
    assert [policy.capacity(n) for n in (1, 3, 5, 9, 25, 64)] == [1, 4, 6, 12, 32, 64]
    assert policy.capacity_allow_zero(0) == 0


def test_topology_boundaries_prevent_cross_topology_padding():
    policy = ReplayBucketPolicy.with_topology_boundaries(64, [5, 6, 10, 12, 18])
    assert 0 not in policy.buckets()
    assert [policy.capacity(n) for n in (5, 9, 10, 11, 17, 18)] == [5, 9, 11, 11, 17, 20]
    assert ReplayBucketPolicy.with_topology_boundaries(6, [1]).buckets() == [1, 2, 4, 6]
    policy = ReplayBucketPolicy.with_topology_boundaries(8, [6])
    assert policy.buckets() == [1, 2, 4, 5, 6, 8]
    assert [policy.capacity(n) for n in (5, 6, 7)] == [5, 6, 8]


def test_default_policy_keeps_inactive_lanes_at_or_below_one_quarter():
    policy = ReplayBucketPolicy(256)
    for active in range(1, 257):
        total = policy.capacity(active)
        assert (total - active) * 4 <= total, (active, total)


def test_capacity_rejects_active_work_above_limit():
    with pytest.raises(KhmError, match="replay active work exceeds capacity"):
        ReplayBucketPolicy(6).capacity(7)
    with pytest.raises(KhmError, match="replay bucket requires active work"):
        ReplayBucketPolicy(6).capacity(0)
