"""Executor-side selector: exact vectors and invariants of the reference's host-only tests
(crates/inference-executor-metal/src/attn/gqa/sdpa_test.rs), through the C ABI."""
import itertools

import pytest

from khalamari_amd import sdpa
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, KhmError
from khalamari_amd.selector import GQAReplayBucketPolicy, RequestShape, Selector
from khalamari_amd.sliced_kv import Layout


def _cfg(hq, hkv, d, tpp, dtype=DTYPE_BF16):
    return sdpa.Config(dtype, hq, hkv, d, tpp)


D256 = _cfg(24, 4, 256, 16)


def _selector_for(config):
    registry = sdpa.Registry(config)
    return Selector.new(registry, 128, 128, 128 * registry.max_q_tokens_per_map_task())


def _selection(token_indices, request_tokens, config=D256):
    cu = [0] + list(itertools.accumulate(request_tokens))
    shapes = RequestShape.from_batch(token_indices, cu)
    return _selector_for(config).select(shapes, GQAReplayBucketPolicy(128, 128), cu[-1])


def _is_sliced_kv(selection):
    return selection.variant().map_kind == sdpa.MAP_SLICED_KV


def test_request_shapes_from_batch():
    assert RequestShape.from_batch([7, 20], [0, 2, 5]) == [RequestShape(7, 2), RequestShape(20, 3)]
    with pytest.raises(KhmError, match="GQA requests must contain Q tokens"):
        RequestShape.from_batch([7, 20], [0, 2, 2])
    with pytest.raises(KhmError, match="nondecreasing"):
        RequestShape.from_batch([7, 20], [0, 3, 2])
    with pytest.raises(KhmError, match="must fit u32"):
        RequestShape.from_batch([0xFFFFFFFF], [0, 1])


def test_fixed_slices_cover_ragged_causal_ranges():
    # sdpa_test.rs:302-355
    config = _cfg(12, 2, 128, 16)
    variant = sdpa.ExecutionVariant.sliced_q(config, sdpa.MAP_Q_TOKENS_AND_HEADS, 4, 16, 6)
    selector = Selector.new(sdpa.Registry.from_variants(config, [variant]), 16, 64, 256)
    requests = RequestShape.from_batch([120, 2], [0, 5, 8])
    policy = GQAReplayBucketPolicy(16, 64)
    selection = selector.select_partitioned(variant, 64, False, requests, policy, 8)
    assert selection.q_token_ranges() == [(0, 0, 4, 124), (0, 4, 5, 125), (1, 5, 8, 5)]
    assert selection.map_task_templates() == [(0, 0, 64), (0, 64, 124), (1, 0, 64), (1, 64, 125), (2, 0, 5)]
    assert selection.cu_partial_outputs_by_q_token_range() == [0, 2, 4, 5]
    assert selection.metrics().max_kv_iterations_per_split == 4
    assert not selection.direct_output()
    selection = selector.select_partitioned(variant, 65, False, requests, policy, 8)
    assert selection.map_task_templates() == [(0, 0, 65), (0, 65, 124), (1, 0, 65), (1, 65, 125), (2, 0, 5)]
    assert selection.cu_partial_outputs_by_q_token_range() == [0, 2, 4, 5]
    assert selection.metrics().max_kv_iterations_per_split == 5
    assert selection.metrics().num_scheduled_qk_token_pairs == 1216
    assert selection.metrics().num_active_qk_token_pairs == 768


def test_direct_output_preserves_padded_range_identity_without_partials():
    # sdpa_test.rs:357-385
    config = _cfg(1, 1, 128, 16)
    variant = sdpa.ExecutionVariant.sliced_q_per_head(config, 1, 16, 1)
    selector = Selector.new(sdpa.Registry.from_variants(config, [variant]), 9, 64, 1)
    requests = RequestShape.from_batch([64, 2], [0, 7, 9])
    selection = selector.select_partitioned(variant, 71, True, requests, GQAReplayBucketPolicy(9, 64), 9)
    shape = selection.replay_shape()
    assert selection.direct_output()
    assert shape.num_q_token_tiles == 9 and shape.num_sdpa_map_task_templates == 9
    assert shape.num_total_q_token_tiles == shape.num_total_sdpa_map_task_templates == 9
    assert selection.metrics().num_active_partial_state_groups == 0
    assert selection.metrics().num_replay_reserved_partial_state_groups == 0
    for (_, _, _, visible), (_, begin, end) in zip(selection.q_token_ranges(), selection.map_task_templates()):
        assert (begin, end) == (0, visible)
    with pytest.raises(KhmError, match="GQA direct output requires an unsplit KV range"):
        selector.select_partitioned(variant, 70, True, requests, GQAReplayBucketPolicy(9, 64), 9)


def test_selector_preserves_measured_d256_page16_crossovers():
    # sdpa_test.rs:387-395
    for tokens, context in [(1, 65536), (2, 65536), (4, 128), (8, 128), (25, 32)]:
        assert _is_sliced_kv(_selection([context], [tokens]))
    for tokens, context in [(4, 512), (8, 512), (16, 128), (25, 128), (64, 0)]:
        assert not _is_sliced_kv(_selection([context], [tokens]))


def test_selector_preserves_other_profile_selection():
    # sdpa_test.rs:397-437
    shapes = RequestShape.from_batch([0] * 4, [0, 2, 4, 6, 8])
    policy = GQAReplayBucketPolicy(128, 128)
    v = _selector_for(_cfg(24, 4, 256, 32)).select(shapes, policy, 8).variant()
    assert (v.map_max_q_tokens, v.map_max_q_heads) == (8, 3)
    v = _selector_for(_cfg(32, 4, 128, 16)).select(shapes, policy, 8).variant()
    assert (v.map_max_q_tokens, v.map_max_q_heads) == (8, 8)
    v = _selector_for(_cfg(32, 4, 256, 4)).select(shapes, policy, 8).variant()
    assert v.map_max_q_tokens == 1


def test_selector_prices_request_local_tail_ranges():
    # sdpa_test.rs:439-445
    assert _is_sliced_kv(_selection([65536] * 8, [1] * 8))
    assert _is_sliced_kv(_selection([1024, 65536], [64, 1]))
    assert _is_sliced_kv(_selection([65536, 1024], [1, 8]))
    assert not _is_sliced_kv(_selection([65536, 65536], [8, 1]))


def test_selection_materializes_current_sliced_q_capacity_and_metrics():
    # sdpa_test.rs:447-470
    assert _is_sliced_kv(_selection([1024, 65536], [64, 1]))
    mixed = _selection([8192, 65536], [64, 64])
    cu = mixed.cu_partial_outputs_by_q_token_range()
    assert [b - a for a, b in zip(cu, cu[1:])] == [2] * 8 + [14] * 8
    selection = _selection([65536], [25])
    assert not _is_sliced_kv(selection)
    assert len(selection.q_token_ranges()) == 4
    assert len(selection.map_task_templates()) == 128
    assert selection.replay_shape().num_total_sdpa_map_task_templates == 128
    m = selection.metrics()
    assert m.num_active_partial_state_groups == 800
    assert m.num_active_partial_states == 800 * 24
    assert m.num_reserved_partial_state_groups == 1024
    assert m.num_replay_reserved_partial_state_groups == 1024


def _assert_contiguous_cover(selection):
    cu = selection.cu_partial_outputs_by_q_token_range()
    templates = selection.map_task_templates()
    for index, (_, _, _, visible) in enumerate(selection.q_token_ranges()):
        own = templates[cu[index]:cu[index + 1]]
        assert own and own[0][1] == 0 and own[-1][2] == visible
        assert all(t[0] == index for t in own)
        assert all(a[2] == b[1] for a, b in zip(own, own[1:]))


def test_selection_map_tasks_cover_each_visible_kv_range_once():
    # sdpa_test.rs:472-509
    for histories, q_tokens in [([1024], [25]), ([8192, 65536], [64, 64]), ([0], [1]), ([0], [128]), ([65536] * 128, [1] * 128)]:
        selection = _selection(histories, q_tokens)
        stage = selection.variant().map_kv_tokens_per_iteration
        iterations = sum(-(-visible // stage) for (_, _, _, visible) in selection.q_token_ranges())
        assert len(selection.map_task_templates()) == min(iterations, 128)
        _assert_contiguous_cover(selection)


def test_dense_prefill_kv32_preserves_request_ranges_and_replay_capacity():
    # sdpa_test.rs:511-557
    registry = sdpa.Registry(D256)
    selector = Selector.new(registry, 2048, 2048, 2048 * registry.max_q_tokens_per_map_task())
    policy = GQAReplayBucketPolicy(2048, 2048)
    for histories, cu in [([0], [0, 1024]), ([4096], [0, 1024]), ([0, 16384], [0, 512, 1024])]:
        selection = selector.select(RequestShape.from_batch(histories, cu), policy, 2048)
        assert selection.variant().map_kv_tokens_per_iteration == 32
        assert selection.replay_shape().num_tokens == 1024
        assert selection.replay_shape().num_total_tokens == 2048
        assert len(selection.map_task_templates()) == 256
        _assert_contiguous_cover(selection)
    short = selector.select(RequestShape.from_batch([4096], [0, 256]), policy, 2048)
    assert short.variant().map_kv_tokens_per_iteration == 16
    decode = selector.select(RequestShape.from_batch([4096] * 1024, list(range(1025))), policy, 2048)
    assert decode.variant().map_max_q_tokens == 1


def test_map_capacity_preserves_token_domain_and_replay_padding():
    # sdpa_test.rs:559-587
    config = _cfg(1, 1, 128, 8)
    variant = sdpa.ExecutionVariant.sliced_kv(config, 64, 128, 1)
    selector = Selector.new(sdpa.Registry.from_variants(config, [variant]), 4, 32, 32)
    policy = GQAReplayBucketPolicy(4, 32)
    selection = selector.select(RequestShape.from_batch([1088], [0, 1]), policy, 2)
    shape = selection.replay_shape()
    assert selector.limits().max_tokens == 4
    assert shape.as_tuple() == (1, 2, 1, 1, 18, 20, True)
    assert selection.metrics().num_replay_reserved_partial_state_groups == 20
    assert selection.map_task_templates()[-1] == (0, 1088, 1089)
    with pytest.raises(KhmError):
        selector.select(RequestShape.from_batch([0], [0, 5]), policy, 4)


def test_partial_state_capacity_includes_replay_padding():
    # sdpa_test.rs:589-601
    config = _cfg(1, 1, 128, 8)
    variant = sdpa.ExecutionVariant.sliced_kv(config, 64, 128, 1)
    selector = Selector.new(sdpa.Registry.from_variants(config, [variant]), 4, 32, 18)
    with pytest.raises(KhmError, match="GQA SDPA replay exceeds its partial-state-group capacity"):
        selector.select(RequestShape.from_batch([1088], [0, 1]), GQAReplayBucketPolicy(4, 32), 2)


def test_total_token_count_rejects_overflows():
    # sdpa_test.rs:603-613
    shapes = RequestShape.from_batch([0], [0, 5])
    with pytest.raises(KhmError, match="GQA active token count must not exceed the total token count"):
        _selector_for(D256).select(shapes, GQAReplayBucketPolicy(128, 128), 4)
    with pytest.raises(KhmError, match="GQA total token count must not exceed the metadata capacity"):
        _selector_for(D256).select(shapes, GQAReplayBucketPolicy(128, 128), 129)
    with pytest.raises(KhmError, match="must match the SDPA token capacity"):
        _selector_for(D256).select(shapes, GQAReplayBucketPolicy(64, 128), 5)


def test_partition_envelope_keeps_variant_maps_and_token_tiles_coupled():
    # sdpa_test.rs:185-216
    single = sdpa.ExecutionVariant.sliced_kv(D256, 256, 128, 6)
    sliced_q = sdpa.ExecutionVariant.sliced_q_per_head(D256, 8, 16, 6)
    registry = sdpa.Registry.from_variants(D256, [single, sliced_q])
    selector = Selector.for_partitions(registry, 128, 8, lambda v: -(-32768 // 512))
    assert selector.limits().max_map_task_templates == 8192
    assert selector.limits().partial_state_group_capacity == 12288
    selector = Selector.for_partitions(registry, 128, 8, lambda v: 64 if v.map_kind == sdpa.MAP_SLICED_KV else 8)
    assert selector.limits().max_map_task_templates == 8192
    assert selector.limits().partial_state_group_capacity == 8192


def _compositions(total, parts):
    if parts == 1:
        yield [total]
        return
    for first in range(1, total - parts + 2):
        for rest in _compositions(total - first, parts - 1):
            yield [first] + rest


def test_partition_envelope_covers_positive_request_compositions():
    # sdpa_test.rs:218-282 (token capacities up to 10 keep the CPU suite short)
    config = _cfg(1, 1, 128, 16)
    variants = [sdpa.ExecutionVariant.sliced_q_per_head(config, tile, 16, 1) for tile in (1, 2, 4, 8, 16, 32)]
    registry = sdpa.Registry.from_variants(config, variants)
    for max_tokens in range(1, 11):
        for max_requests in range(1, 5):
            selector = Selector.for_partitions(registry, max_tokens, max_requests, lambda v: -(-130 // 64))
            limits = selector.limits()
            policy = GQAReplayBucketPolicy(max_tokens, limits.max_map_task_templates)
            observed = [0] * 6
            for total in range(1, max_tokens + 1):
                for requests in range(1, min(max_requests, total) + 1):
                    for tokens in _compositions(total, requests):
                        shapes = [RequestShape(130 - n, n) for n in tokens]
                        for i, variant in enumerate(variants):
                            selection = selector.select_partitioned(variant, 64, False, shapes, policy, total)
                            shape = selection.replay_shape()
                            observed[i] = max(observed[i], shape.num_q_token_tiles)
                            assert shape.num_total_sdpa_map_task_templates <= limits.max_map_task_templates
                            assert selection.metrics().num_replay_reserved_partial_state_groups <= limits.partial_state_group_capacity
            requests = min(max_requests, max_tokens)
            for i, variant in enumerate(variants):
                assert observed[i] == requests + (max_tokens - requests) // variant.map_max_q_tokens


def test_partition_envelope_rejects_map_count_overflow_before_allocation():
    # sdpa_test.rs:284-300
    config = _cfg(1, 1, 128, 16)
    variant = sdpa.ExecutionVariant.sliced_kv(config, 128, 128, 1)
    with pytest.raises(KhmError, match="GQA partition Map task-template count must fit u32"):
        Selector.for_partitions(sdpa.Registry.from_variants(config, [variant]), 0xFFFFFFFF, 1, lambda v: 2)


# ---- lookup route: the reference's table is fitted to an M3 Max and is replaced; its invariants are kept ----

def test_lookup_preserves_f32_execution_capability():
    # sdpa_test.rs:39-76: io dtypes without a sliced-Q kernel keep the sliced-KV route
    for head_dim in (128, 256):
        config = _cfg(24, 4, head_dim, 16, DTYPE_F32)
        selector = Selector.for_lookup(config, 128, Layout(4, 1, 1024, 1))
        policy = GQAReplayBucketPolicy(128, selector.limits().max_map_task_templates)
        for history in (0, 4096):
            for q in (1, 8):
                selection = selector.select([RequestShape(history, q)], policy, q)
                assert _is_sliced_kv(selection)
                assert sdpa.supports(selection.variant(), config)


def test_lookup_keeps_single_query_requests_on_the_split_kv_path():
    # sdpa_test.rs:78-118 (the short-context direct route is M3 policy; here decode is always Map/Reduce)
    for hq, hkv, d in [(24, 4, 256), (16, 2, 256), (40, 8, 128)]:
        config = _cfg(hq, hkv, d, 16)
        selector = Selector.for_lookup(config, 128, Layout(8, 1, 128, 1))
        policy = GQAReplayBucketPolicy(128, selector.limits().max_map_task_templates)
        for history in (0, 31, 32, 128, 384, 511, 512, 1024):
            for requests in (1, 4, 8):
                result = selector.select([RequestShape(history, 1)] * requests, policy, requests)
                assert _is_sliced_kv(result) and not result.direct_output()
                assert result.variant().map_max_q_heads == hq // hkv
                assert sdpa.has_kernel(config, result.variant())
                _assert_contiguous_cover(result)


def test_lookup_covers_ragged_queries_and_continuous_context_within_replay_capacity():
    # sdpa_test.rs:120-183
    for dim, ratio in [(128, 1), (128, 6), (128, 8), (128, 12), (256, 6), (256, 8), (256, 12), (256, 32)]:
        config = _cfg(4 * ratio, 4, dim, 16)
        selector = Selector.for_lookup(config, 2048, Layout(8, 1, 16400, 1))
        limits = selector.limits()
        policy = GQAReplayBucketPolicy(2048, limits.max_map_task_templates)
        for history in (0, 63, 64, 255, 256, 511, 512, 513, 1023, 2048, 4095, 4096, 4097, 8191, 16383, 32768, 65535, 98317, 131073, 262144):
            for queries in (1, 2, 3, 5, 8, 12, 32, 64, 256):
                for requests in (1, 2, 8):
                    shapes = [RequestShape(history - min(history, i), queries - min(i, queries - 1)) for i in range(requests)]
                    result = selector.select(shapes, policy, 2048)
                    assert result.replay_shape().num_total_sdpa_map_task_templates <= limits.max_map_task_templates
                    assert result.metrics().num_replay_reserved_partial_state_groups <= limits.partial_state_group_capacity
                    assert result.variant() in selector.variants()
                    assert sdpa.has_kernel(config, result.variant())
                    _assert_contiguous_cover(result)


def test_lookup_fills_the_chip_for_the_benchmark_shapes():
    # 32 decode requests, contexts 512..8192, Hq64/Hkv8: enough blocks for 256 compute units, slices >= 256 tokens
    config = _cfg(64, 8, 128, 16)
    selector = Selector.for_lookup(config, 64, Layout(32, 1, 512, 1))
    policy = GQAReplayBucketPolicy(64, selector.limits().max_map_task_templates)
    shapes = [RequestShape(511 + 240 * i, 1) for i in range(32)]
    result = selector.select(shapes, policy, 32)
    blocks = len(result.map_task_templates()) * 8
    assert blocks >= 512
    assert min(end - begin for (_, begin, end) in result.map_task_templates() if end - begin) >= 1
    assert max(end - begin for (_, begin, end) in result.map_task_templates()) >= 256
    # a dense 2048-token prefill chunk per request needs no KV split: direct output
    prefill = selector_prefill = Selector.for_lookup(config, 16384, Layout(8, 1, 2048, 1))
    policy = GQAReplayBucketPolicy(16384, prefill.limits().max_map_task_templates)
    result = selector_prefill.select([RequestShape(4096, 2048)] * 8, policy, 16384)
    assert result.direct_output()


def test_lookup_hands_out_exactly_the_block_budget_in_equal_splits():
    """A batch of 16 speculative blocks (q_len 2..5 on contexts of 4096..32768 tokens, Hq64/Hkv8): the verify kernels hold a
    whole number of blocks per compute unit, so the route must not exceed 1024 blocks, and the splits of all ranges end up
    about equally long, in whole 64-token iterations."""
    config = _cfg(64, 8, 128, 16)
    histories = [4096 + 1791 * i for i in range(16)]
    q_lens = [2 + i % 4 for i in range(16)]
    selector = Selector.for_lookup(config, sum(q_lens), Layout(16, 1, 2064, 1))
    policy = GQAReplayBucketPolicy(selector.limits().max_tokens, selector.limits().max_map_task_templates)
    result = selector.select([RequestShape(h, q) for h, q in zip(histories, q_lens)], policy, sum(q_lens))
    templates = result.map_task_templates()
    assert not result.direct_output()
    assert len(templates) * 8 == 1024
    lengths = [end - begin for (_, begin, end) in templates]
    assert max(lengths) <= 2 * min(lengths) and min(lengths) >= 256
    assert all(begin % 64 == 0 for (_, begin, _) in templates)
    _assert_contiguous_cover(result)
    # short contexts are not cut below 256 tokens per split on average, and an unsplit sliced-Q batch writes its output directly
    short = selector.select([RequestShape(300, 3)] * 4, policy, 12)
    assert short.direct_output() and len(short.map_task_templates()) == len(short.q_token_ranges())
