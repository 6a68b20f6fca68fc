"""Host side of block (DFlash2 proposal) attention against the reference's exact integer vectors: capacity
(attn/bidi_block_gqa/capacity.rs:55-62), selector (attn/bidi_block_gqa/sdpa.rs:116-139), core metadata
(bidi_block_gqa_core.rs:170-206) and GPU metadata (attn/bidi_block_gqa/metadata.rs:380-527).  CPU only."""
import numpy as np
import pytest

from khalamari_amd import _lib, bidi_block_metadata as bbm, sdpa
from khalamari_amd._lib import DTYPE_BF16

U32_MAX = 0xFFFFFFFF


def _small_config():
    """`config()` of metadata.rs:597-605."""
    return sdpa.Config(DTYPE_BF16, 2, 1, 128, 8)


def _per_head_variant():
    return sdpa.ExecutionVariant.sliced_q_per_head(_small_config(), 8, 16, 2)


def test_capacity_reserves_history_and_block_partials():
    capacity = bbm.capacity(3, 7, 8)
    assert capacity.max_tokens == 21
    assert capacity.max_q_token_ranges == 3
    assert capacity.max_sdpa_map_task_templates == 32
    assert capacity.max_sdpa_partial_state_groups == 256


def _selector_config(head_dim, tokens_per_page):
    return sdpa.Config(DTYPE_BF16, 40, 8, head_dim, tokens_per_page)


def test_selector_uses_q_tile_only_when_it_reuses_history():
    sliced_kv, _ = bbm.select(_selector_config(128, 16), 2, 1)
    sliced_q, capacity = bbm.select(_selector_config(128, 16), 2, 7)
    assert sliced_kv.map_max_q_tokens == 1
    assert sliced_q.map_max_q_tokens == 8
    assert capacity.max_q_tokens == 8


def test_selector_keeps_sliced_kv_for_unsupported_tiled_profile():
    variant, capacity = bbm.select(_selector_config(128, 4), 2, 7)
    assert variant.map_max_q_tokens == 1 and capacity.max_q_tokens == 1


def test_selector_minimizes_history_kv_loads():
    variant, _ = bbm.select(_selector_config(256, 32), 2, 7)
    assert variant.map_max_q_heads == 5


def test_block_metadata_uses_history_end_as_first_query_row():
    m = bbm.build([2, 9], [11, 12, 13, 20, 21, 22], [(0, 11)] * 3 + [(4, 20)] * 3, 3, _per_head_variant(), 8)
    assert m.req_slots.tolist() == [2, 2, 2, 9, 9, 9]
    assert m.flat_token_indices.tolist() == [11, 12, 13, 20, 21, 22]
    assert m.visible_kv_token_ranges[:, 0].tolist() == [0, 0, 0, 4, 4, 4]
    assert m.visible_kv_token_ranges[:, 1].tolist() == [11, 11, 11, 20, 20, 20]


def test_block_metadata_rejects_what_the_reference_rejects():
    variant = _per_head_variant()
    with pytest.raises(_lib.KhmError, match="unique request slots"):
        bbm.build([2, 2], [11, 12, 13, 20, 21, 22], [(0, 11)] * 6, 3, variant, 8)
    with pytest.raises(_lib.KhmError, match="nonempty half-open ranges"):
        bbm.build([2], [11, 12, 13], [(11, 11), (0, 11), (0, 11)], 3, variant, 8)
    with pytest.raises(_lib.KhmError, match="one query-token index per block row"):
        bbm.build([2], [11, 12], [(0, 11)] * 3, 3, variant, 8)
    with pytest.raises(_lib.KhmError, match="active BiDiBlockGQA requests"):
        bbm.build([2], [11, 12, 13], [(0, 11)] * 3, 3, variant, 8, num_active_requests=2)


def test_block_metadata_preserves_per_query_history_ranges():
    m = bbm.build([2], [11, 12, 13], [(0, 11), (1, 11), (2, 11)], 3, _per_head_variant(), 8)
    assert m.visible_kv_token_ranges.tolist() == [[0, 11], [1, 11], [2, 11]]


def test_metadata_materializes_tiled_history_and_block_partials():
    capacity = bbm.capacity(2, 3, 8)
    m = bbm.build([3, 7], [11, 12, 13, 20, 21, 22], [(0, 11)] * 3 + [(3, 20)] * 3, 3, _per_head_variant(), capacity.max_sdpa_map_task_templates)
    shape = m.replay_shape
    assert shape.num_tokens == 6 and shape.num_q_token_tiles == 2 and shape.num_total_sdpa_map_task_templates == 8
    assert m.visible_kv_token_ranges.reshape(-1).tolist() == [0, 11, 0, 11, 0, 11, 3, 20, 3, 20, 3, 20]
    assert m.q_token_ranges.reshape(-1).tolist() == [0, 3, 3, 6]
    assert m.cu_sdpa_partial_outputs.tolist() == [0, 2, 5]
    # one history task for the 11-token range, two for the 17-token one, each followed by the block-partial placeholder
    assert m.sdpa_map_task_templates.tolist() == [[0, 0, 11], [U32_MAX] * 3, [1, 3, 19], [1, 19, 20], [U32_MAX] * 3] + [[U32_MAX] * 3] * 3
    assert bool(shape.reduce_sdpa_partial_outputs)


def test_long_history_is_partitioned_without_growing_static_scratch():
    anchor = 262_144
    m = bbm.build([1], list(range(anchor, anchor + 6)), [(0, anchor)] * 6, 6, _per_head_variant(), 16)
    block_task = int(m.cu_sdpa_partial_outputs[1]) - 1
    history = m.sdpa_map_task_templates[:block_task]
    assert history[0][1] == 0 and history[-1][2] == anchor
    assert all(history[i][2] == history[i + 1][1] for i in range(len(history) - 1))
    assert m.cu_sdpa_partial_outputs.tolist() == [0, 16]
    assert m.replay_shape.num_total_sdpa_map_task_templates == 16


def test_q_tile_uses_history_union_and_preserves_per_query_masks():
    capacity = bbm.capacity(1, 3, 8)
    m = bbm.build([3], [20, 21, 22], [(0, 20), (1, 20), (2, 20)], 3, _per_head_variant(), capacity.max_sdpa_map_task_templates)
    assert m.replay_shape.num_q_token_tiles == 1
    assert m.visible_kv_token_ranges.reshape(-1).tolist() == [0, 20, 1, 20, 2, 20]
    assert m.sdpa_map_task_templates[0][1] == 0 and m.sdpa_map_task_templates[0][2] <= 20


def test_active_request_prefix_shrinks_the_replay_shape_only():
    """update_with_active_requests (metadata.rs:91-141): arrays cover every request, the shape the active ones."""
    m = bbm.build([3, 7], [11, 12, 13, 20, 21, 22], [(0, 11)] * 3 + [(3, 20)] * 3, 3, _per_head_variant(), 8, num_active_requests=1)
    assert m.replay_shape.as_tuple() == (3, 6, 1, 2, 2, 8, True)
    assert m.cu_sdpa_partial_outputs.tolist() == [0, 2, 5]


def _spec_decode_block(anchors, block_size, history_window):
    """`spec_decode_block` (metadata.rs:529-549): row i of a block sits at anchor + i and sees the window before the anchor."""
    indices, ranges = [], []
    for anchor in anchors:
        for offset in range(block_size):
            position = anchor + offset
            indices.append(position)
            ranges.append((max(position + 1 - history_window, 0), anchor))
    return indices, ranges


@pytest.mark.parametrize("anchors,spec,accepted,block_size,window", [
    ([10], [7], [a], 7, U32_MAX) for a in range(8)] + [
    ([10, 31], [7, 7], [0, 5], 7, U32_MAX),
    ([10, 31, 65, 96], [7, 7, 7, 7], [7, 2, 0, 6], 7, U32_MAX),
    ([10, 31, 65, 96], [7, 7, 7, 7], [0, 4, 7, 2], 8, 16),
])
def test_spec_decode_fixed_quota_rewrite_matches_rebuild(anchors, spec, accepted, block_size, window):
    """test_spec_decode_success (metadata.rs:445-527): metadata built for the largest accepted anchors, then rewritten in
    place for the accepted ones with the task counts kept, covers the same history as metadata built from scratch."""
    config = _small_config()
    variant, capacity = bbm.select(config, 4, block_size)
    max_templates = bbm.capacity(len(anchors), block_size, variant.map_max_q_tokens).max_sdpa_map_task_templates
    slots = list(range(len(anchors)))
    accepted_anchors = [a + n for a, n in zip(anchors, accepted)]
    static = bbm.build(slots, *_spec_decode_block([a + n for a, n in zip(anchors, spec)], block_size, window), block_size, variant, max_templates)
    cpu = bbm.build(slots, *_spec_decode_block(accepted_anchors, block_size, window), block_size, variant, max_templates)
    per_iteration, max_q = int(variant.map_kv_tokens_per_iteration), int(variant.map_max_q_tokens)
    ranges_per_request = -(-block_size // max_q)
    tasks, visible = static.sdpa_map_task_templates.copy(), static.visible_kv_token_ranges.copy()
    for request, anchor in enumerate(accepted_anchors):       # rewrite_fixed_quota_for_test (metadata.rs:551-589)
        begin_row = request * block_size
        for offset in range(block_size):
            visible[begin_row + offset] = (max(anchor + offset + 1 - window, 0), anchor)
        for local in range(ranges_per_request):
            q_range = request * ranges_per_request + local
            first_position = anchor + int(static.q_token_ranges[q_range][0]) - begin_row
            history_begin = max(first_position + 1 - window, 0)
            task_begin, task_end = int(static.cu_sdpa_partial_outputs[q_range]), int(static.cu_sdpa_partial_outputs[q_range + 1]) - 1
            count = task_end - task_begin
            iterations = -(-(anchor - history_begin) // per_iteration)
            for k in range(count):
                tasks[task_begin + k] = (q_range, history_begin + (iterations * k // count) * per_iteration,
                                         min(anchor, history_begin + (iterations * (k + 1) // count) * per_iteration))
    assert np.array_equal(visible, cpu.visible_kv_token_ranges)
    assert np.array_equal(static.q_token_ranges, cpu.q_token_ranges)
    for q_range in range(int(cpu.replay_shape.num_q_token_tiles)):
        begin, end = int(static.cu_sdpa_partial_outputs[q_range]), int(static.cu_sdpa_partial_outputs[q_range + 1]) - 1
        cpu_begin, cpu_end = int(cpu.cu_sdpa_partial_outputs[q_range]), int(cpu.cu_sdpa_partial_outputs[q_range + 1]) - 1
        history = tasks[begin:end]
        assert history[0][1] == cpu.sdpa_map_task_templates[cpu_begin][1]
        assert history[-1][2] == cpu.sdpa_map_task_templates[cpu_end - 1][2]
        assert all(task[0] == q_range for task in history)
        assert all(history[i][2] == history[i + 1][1] for i in range(len(history) - 1))
        assert tasks[end].tolist() == [U32_MAX] * 3
