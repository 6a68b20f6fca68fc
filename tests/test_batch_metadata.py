"""GPU metadata ABI: exact uploaded arrays of crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:329-465,
computed with the host form of `GQAMetadataBuffers::update` (no device needed)."""
import numpy as np

from khalamari_amd import batch_metadata, sdpa
from khalamari_amd._lib import DTYPE_BF16
from khalamari_amd.selector import GQAReplayBucketPolicy, RequestShape, Selector

U32_MAX = 0xFFFFFFFF
CONFIG = sdpa.Config(DTYPE_BF16, 2, 2, 128, 8)


def _selector(max_tokens, variant):
    return Selector.new(sdpa.Registry.from_variants(CONFIG, [variant]), max_tokens, max_tokens, max_tokens * variant.map_max_q_tokens)


def test_map_metadata_capacity_is_independent_of_token_capacity():
    variant = sdpa.ExecutionVariant.sliced_kv(CONFIG, 64, 128, 1)
    selector = Selector.new(sdpa.Registry.from_variants(CONFIG, [variant]), 4, 32, 32)
    selection = selector.select(RequestShape.from_batch([1088], [0, 1]), GQAReplayBucketPolicy(4, 32), 2)
    slots, flat, visible, ranges, templates, cu = batch_metadata.compute([1], [1088], [0, 1], selection, 4, 32)
    shape = selection.replay_shape()
    assert (shape.num_tokens, shape.num_total_tokens) == (1, 2)
    assert (shape.num_sdpa_map_task_templates, shape.num_total_sdpa_map_task_templates) == (18, 20)
    assert slots.size == 4 and templates.size == 32 * 3
    assert flat[0] == 1088
    assert list(visible[:2]) == [0, 1089]
    assert list(templates[18 * 3:20 * 3]) == [U32_MAX] * 6
    assert list(cu[:2]) == [0, 18]


def test_metadata_upload_preserves_current_abi_for_complete_selections():
    shapes = RequestShape.from_batch([7, 20], [0, 2, 5])
    policy = GQAReplayBucketPolicy(8, 8)
    single = sdpa.ExecutionVariant.sliced_kv(CONFIG, 8, 32, 1)
    selection = _selector(8, single).select(shapes, policy, 5)
    slots, flat, visible, ranges, templates, cu = batch_metadata.compute([2, 5], [7, 20], [0, 2, 5], selection, 8, 8)
    assert list(slots[:5]) == [2, 2, 5, 5, 5]
    assert list(flat[:5]) == [7, 8, 20, 21, 22]
    assert list(visible[:10]) == [0, 8, 0, 9, 0, 21, 0, 22, 0, 23]
    assert list(templates[:24]) == [0, 0, 8, 1, 0, 9, 2, 0, 8, 2, 8, 21, 3, 0, 8, 3, 8, 22, 4, 0, 8, 4, 8, 23]
    assert list(cu[:6]) == [0, 1, 2, 4, 6, 8]
    assert selection.replay_shape().as_tuple() == (5, 5, 5, 6, 8, 8, True)

    sliced_q = sdpa.ExecutionVariant.sliced_q_per_head(CONFIG, 8, 8, 1)
    selection = _selector(8, sliced_q).select(shapes, policy, 5)
    slots, flat, visible, ranges, templates, cu = batch_metadata.compute([2, 5], [7, 20], [0, 2, 5], selection, 8, 8)
    assert list(ranges[:4]) == [0, 2, 2, 5]
    assert list(templates[:18]) == [0, 0, 8, 0, 8, 9, 1, 0, 8, 1, 8, 16, 1, 16, 23, U32_MAX, U32_MAX, U32_MAX]
    assert list(cu[:3]) == [0, 2, 5]
    assert selection.replay_shape().as_tuple() == (5, 5, 2, 2, 5, 6, True)
    assert selection.variant() == sliced_q


def test_selection_preserves_non_kv_metadata_tail():
    variant = sdpa.ExecutionVariant.sliced_q_per_head(CONFIG, 8, 8, 1)
    selection = _selector(12, variant).select(RequestShape.from_batch([0, 0, 0], [0, 4, 8, 9]), GQAReplayBucketPolicy(12, 12), 12)
    slots, flat, visible, ranges, templates, cu = batch_metadata.compute([2, 5, 7], [0, 0, 0], [0, 4, 8, 9], selection, 12, 12,
                                                                        fill=0x94949494)
    assert selection.replay_shape().as_tuple() == (9, 12, 3, 4, 3, 4, True)
    assert list(visible[18:20]) == [0x94949494] * 2      # beyond the 9 active tokens: untouched
    assert list(ranges[6:8]) == [0x94949494] * 2         # beyond the 3 active ranges: untouched
    assert list(templates[9:12]) == [U32_MAX] * 3        # padded template
    assert cu[4] == 0x94949494                           # beyond ranges + 1: untouched


def test_sliced_kv_selection_leaves_q_token_ranges_untouched():
    variant = sdpa.ExecutionVariant.sliced_kv(CONFIG, 8, 32, 1)
    selection = _selector(8, variant).select(RequestShape.from_batch([7], [0, 2]), GQAReplayBucketPolicy(8, 8), 2)
    arrays = batch_metadata.compute([0], [7], [0, 2], selection, 8, 8, fill=0xA5A5A5A5)
    assert np.all(arrays[batch_metadata.Q_TOKEN_RANGES] == 0xA5A5A5A5)
