"""Mirror of the executor-side selector (crates/inference-executor-metal/src/attn/gqa/sdpa.rs):
`RequestShape`, `Selector`, `Selection`, plus `GQAReplayBucketPolicy` (attn/gqa/batch_metadata.rs:69-96)."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from ._lib import (GqaReplayShape, MapTaskTemplate, PageTableLayout, QTokenRange, SdpaVariant, SelectionMetrics,
                   SelectorLimits)
from ._lib import RequestShape as _CRequestShape
from .sdpa import Config, Registry


@dataclass(frozen=True)
class RequestShape:
    num_history_tokens: int
    num_q_tokens: int

    @staticmethod
    def from_batch(token_indices, cu_tokens):
        n = len(token_indices)
        if len(cu_tokens) != n + 1:
            raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "cu_tokens must hold one more entry than token_indices")
        out = (_CRequestShape * max(n, 1))()
        _lib.check(_lib.lib().khm_request_shapes_from_batch((ctypes.c_uint32 * n)(*token_indices),
                                                            (ctypes.c_uint32 * (n + 1))(*cu_tokens), n, out))
        return [RequestShape(out[i].num_history_tokens, out[i].num_q_tokens) for i in range(n)]


@dataclass(frozen=True)
class GQAReplayBucketPolicy:
    max_tokens: int
    max_map_task_templates: int


class Selection:
    def __init__(self, handle):
        self._handle = handle

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None and getattr(_lib, "_lib", None) is not None:
            _lib._lib.khm_selection_destroy(handle)
            self._handle = None

    def variant(self) -> SdpaVariant:
        out = SdpaVariant()
        _lib.check(_lib.lib().khm_selection_variant(self._handle, ctypes.byref(out)))
        return out

    def direct_output(self) -> bool:
        return bool(_lib.lib().khm_selection_direct_output(self._handle))

    def replay_shape(self) -> GqaReplayShape:
        out = GqaReplayShape()
        _lib.check(_lib.lib().khm_selection_replay_shape(self._handle, ctypes.byref(out)))
        return out

    def metrics(self) -> SelectionMetrics:
        out = SelectionMetrics()
        _lib.check(_lib.lib().khm_selection_metrics_get(self._handle, ctypes.byref(out)))
        return out

    def q_token_ranges(self):
        """[(request_index, flat_begin, flat_end, num_visible_kv_tokens)]"""
        n = _lib.lib().khm_selection_num_q_token_ranges(self._handle)
        array = (QTokenRange * max(n, 1))()
        _lib.check(_lib.lib().khm_selection_q_token_ranges(self._handle, array, n))
        return [(array[i].request_index, array[i].flat_q_token_begin, array[i].flat_q_token_end,
                 array[i].num_visible_kv_tokens) for i in range(n)]

    def map_task_templates(self):
        """[(q_token_range_index, kv_begin, kv_end)]"""
        n = _lib.lib().khm_selection_num_map_task_templates(self._handle)
        array = (MapTaskTemplate * max(n, 1))()
        _lib.check(_lib.lib().khm_selection_map_task_templates(self._handle, array, n))
        return [(array[i].q_token_range_index, array[i].kv_token_begin, array[i].kv_token_end) for i in range(n)]

    def cu_partial_outputs_by_q_token_range(self):
        n = _lib.lib().khm_selection_num_q_token_ranges(self._handle) + 1
        array = (ctypes.c_uint32 * n)()
        _lib.check(_lib.lib().khm_selection_cu_partial_outputs(self._handle, array, n))
        return list(array)


def _shapes(request_shapes):
    n = len(request_shapes)
    array = (_CRequestShape * max(n, 1))()
    for i, shape in enumerate(request_shapes):
        array[i] = _CRequestShape(shape.num_history_tokens, shape.num_q_tokens)
    return array, n


class Selector:
    def __init__(self, handle, config: Config):
        self._handle = handle
        self._config = config

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None and getattr(_lib, "_lib", None) is not None:
            _lib._lib.khm_selector_destroy(handle)
            self._handle = None

    @staticmethod
    def new(registry: Registry, max_tokens: int, max_map_task_templates: int, partial_state_group_capacity: int) -> "Selector":
        variants = registry.variants()
        array = (SdpaVariant * len(variants))(*variants)
        handle = ctypes.c_void_p()
        c = registry.config().c()
        _lib.check(_lib.lib().khm_selector_create(ctypes.byref(c), array, len(variants), ctypes.c_uint64(max_tokens),
                                                  ctypes.c_uint64(max_map_task_templates),
                                                  ctypes.c_uint64(partial_state_group_capacity), ctypes.byref(handle)))
        return Selector(handle, registry.config())

    @staticmethod
    def for_partitions(registry: Registry, max_tokens: int, max_requests: int, max_kv_splits) -> "Selector":
        variants = registry.variants()
        array = (SdpaVariant * len(variants))(*variants)
        splits = (ctypes.c_uint32 * len(variants))(*[max_kv_splits(v) for v in variants])
        handle = ctypes.c_void_p()
        c = registry.config().c()
        _lib.check(_lib.lib().khm_selector_create_for_partitions(ctypes.byref(c), array, splits, len(variants),
                                                                 ctypes.c_uint32(max_tokens), ctypes.c_uint32(max_requests),
                                                                 ctypes.byref(handle)))
        return Selector(handle, registry.config())

    @staticmethod
    def for_lookup(config: Config, max_tokens: int, layout) -> "Selector":
        handle = ctypes.c_void_p()
        c = config.c()
        l = layout.c() if hasattr(layout, "c") else PageTableLayout(*layout)
        _lib.check(_lib.lib().khm_selector_create_for_lookup(ctypes.byref(c), ctypes.c_uint64(max_tokens), ctypes.byref(l),
                                                             ctypes.byref(handle)))
        return Selector(handle, config)

    def limits(self) -> SelectorLimits:
        out = SelectorLimits()
        _lib.check(_lib.lib().khm_selector_limits_get(self._handle, ctypes.byref(out)))
        return out

    def variants(self):
        count = ctypes.c_uint32()
        _lib.check(_lib.lib().khm_selector_variants(self._handle, None, 0, ctypes.byref(count)))
        array = (SdpaVariant * count.value)()
        _lib.check(_lib.lib().khm_selector_variants(self._handle, array, count.value, ctypes.byref(count)))
        return [SdpaVariant.from_buffer_copy(array[i]) for i in range(count.value)]

    def select(self, request_shapes, policy: GQAReplayBucketPolicy, num_total_tokens: int) -> Selection:
        array, n = _shapes(request_shapes)
        handle = ctypes.c_void_p()
        _lib.check(_lib.lib().khm_selector_select(self._handle, array, n, ctypes.c_uint32(policy.max_tokens),
                                                  ctypes.c_uint32(policy.max_map_task_templates),
                                                  ctypes.c_uint32(num_total_tokens), ctypes.byref(handle)))
        return Selection(handle)

    def select_partitioned(self, variant: SdpaVariant, kv_slice: int, direct_output: bool, request_shapes,
                           policy: GQAReplayBucketPolicy, num_total_tokens: int) -> Selection:
        array, n = _shapes(request_shapes)
        handle = ctypes.c_void_p()
        _lib.check(_lib.lib().khm_selector_select_partitioned(
            self._handle, ctypes.byref(variant), ctypes.c_uint32(kv_slice), 1 if direct_output else 0, array, n,
            ctypes.c_uint32(policy.max_tokens), ctypes.c_uint32(policy.max_map_task_templates),
            ctypes.c_uint32(num_total_tokens), ctypes.byref(handle)))
        return Selection(handle)
