"""Mirror of the host side of block (DFlash2 proposal) attention: `BiDiBlockGQAMetadata` (bidi_block_gqa_core.rs:66-139),
`BiDiBlockGQACapacity` (attn/bidi_block_gqa/capacity.rs:7-48), `bidi_block_gqa::sdpa::Selector` (sdpa.rs:46-110) and
`BiDiBlockGQAMetadataBuffers::update` (metadata.rs:87-147,182-375).  All arithmetic lives in the shared library."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence, Tuple

import numpy as np

from . import _lib, sdpa
from ._lib import BidiBlockCapacity, GqaReplayShape, SdpaVariant

U32_MAX = 0xFFFFFFFF


def capacity(max_requests: int, block_size: int, max_q_tokens: int) -> BidiBlockCapacity:
    """`BiDiBlockGQACapacity::new(BiDiBlockCapacity::new(max_requests, block_size), max_q_tokens)`."""
    out = BidiBlockCapacity()
    _lib.check(_lib.lib().khm_bidi_block_capacity_new(max_requests, block_size, max_q_tokens, ctypes.byref(out)))
    return out


def select(config: sdpa.Config, max_requests: int, block_size: int) -> Tuple[SdpaVariant, BidiBlockCapacity]:
    """`Selector::new(Registry::new(config), BiDiBlockCapacity::new(max_requests, block_size)).select()`."""
    cconfig, variant, out = config.c(), SdpaVariant(), BidiBlockCapacity()
    _lib.check(_lib.lib().khm_bidi_block_select(ctypes.byref(cconfig), max_requests, block_size, ctypes.byref(variant), ctypes.byref(out)))
    return variant, out


@dataclass
class BlockMetadata:
    """What `BiDiBlockGQAMetadataBuffers::update` uploads, as host arrays, plus the replay shape of the active prefix."""

    req_slots: np.ndarray
    flat_token_indices: np.ndarray
    visible_kv_token_ranges: np.ndarray
    q_token_ranges: np.ndarray
    sdpa_map_task_templates: np.ndarray
    cu_sdpa_partial_outputs: np.ndarray
    replay_shape: GqaReplayShape


def build(req_slots: Sequence[int], flat_query_token_indices: Sequence[int], visible_history_token_ranges: Sequence[Tuple[int, int]],
          block_size: int, variant: SdpaVariant, max_sdpa_map_task_templates: int, num_active_requests: int = None) -> BlockMetadata:
    """`BiDiBlockGQAMetadata::new(...)` followed by `update_with_active_requests` (all requests active by default)."""
    slots = np.ascontiguousarray(req_slots, dtype=np.uint32)
    num_requests = len(slots)
    num_tokens = num_requests * block_size
    indices = np.ascontiguousarray(flat_query_token_indices, dtype=np.uint32)
    ranges = np.ascontiguousarray(visible_history_token_ranges, dtype=np.uint32).reshape(-1, 2)
    if len(indices) != num_tokens:
        raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "BiDiBlockGQA metadata requires one query-token index per block row")
    if len(ranges) != num_tokens:
        raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "BiDiBlockGQA metadata requires one visible history token range per block row")
    begins, ends = np.ascontiguousarray(ranges[:, 0]), np.ascontiguousarray(ranges[:, 1])
    max_q_tokens = max(int(variant.map_max_q_tokens), 1)
    num_ranges = num_requests * -(-block_size // max_q_tokens)
    out_slots, out_indices = np.zeros(num_tokens, dtype=np.uint32), np.zeros(num_tokens, dtype=np.uint32)
    visible, q_ranges = np.zeros(2 * num_tokens, dtype=np.uint32), np.zeros(2 * num_ranges, dtype=np.uint32)
    templates, cu = np.zeros(3 * max(max_sdpa_map_task_templates, 1), dtype=np.uint32), np.zeros(num_ranges + 1, dtype=np.uint32)
    shape = GqaReplayShape()
    pointer = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))  # noqa: E731
    _lib.check(_lib.lib().khm_bidi_block_metadata_compute(
        pointer(slots), num_requests, pointer(indices), pointer(begins), pointer(ends), block_size, ctypes.byref(variant),
        max_sdpa_map_task_templates, num_requests if num_active_requests is None else num_active_requests, pointer(out_slots),
        pointer(out_indices), pointer(visible), pointer(q_ranges), pointer(templates), pointer(cu), ctypes.byref(shape)))
    total = int(shape.num_total_sdpa_map_task_templates)
    return BlockMetadata(out_slots, out_indices, visible.reshape(-1, 2), q_ranges.reshape(-1, 2), templates[:3 * total].reshape(-1, 3), cu, shape)
