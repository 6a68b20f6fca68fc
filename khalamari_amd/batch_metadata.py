"""Mirror of `GQAMetadataBuffers` (crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:98-326)."""
from __future__ import annotations

import ctypes

import numpy as np

from . import _lib
from ._buffers import stream_handle
from ._lib import Buffer, GqaReplayShape
from .selector import Selection

REQ_SLOTS, FLAT_TOKEN_INDICES, VISIBLE_KV_TOKEN_RANGES, Q_TOKEN_RANGES, SDPA_MAP_TASK_TEMPLATES, CU_SDPA_PARTIAL_OUTPUTS = range(6)


def _u32(values):
    values = [int(v) for v in values]
    return (ctypes.c_uint32 * max(len(values), 1))(*values)


def compute(req_slots, token_indices, cu_tokens, selection: Selection, max_tokens: int, max_map_task_templates: int,
            fill: int = 0):
    """Host form of `update`: returns the six arrays (capacity-sized, `fill` where the update writes nothing)."""
    arrays = [np.full(n, fill, dtype=np.uint32) for n in (max_tokens, max_tokens, 2 * max_tokens, 2 * max_tokens,
                                                         3 * max_map_task_templates, max_tokens + 1)]
    pointers = [a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)) for a in arrays]
    _lib.check(_lib.lib().khm_gqa_metadata_compute(_u32(req_slots), _u32(token_indices), _u32(cu_tokens), len(req_slots),
                                                   selection._handle, *pointers, ctypes.c_uint64(max_tokens),
                                                   ctypes.c_uint64(max_map_task_templates)))
    return arrays


class GQAMetadataBuffers:
    def __init__(self, max_tokens: int, max_map_task_templates: int):
        handle = ctypes.c_void_p()
        _lib.check(_lib.lib().khm_gqa_metadata_create(ctypes.c_uint64(max_tokens), ctypes.c_uint64(max_map_task_templates),
                                                      ctypes.byref(handle)))
        self._handle = handle
        self._max_tokens = max_tokens
        self._max_map_task_templates = max_map_task_templates

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None and getattr(_lib, "_lib", None) is not None:
            _lib._lib.khm_gqa_metadata_destroy(handle)
            self._handle = None

    def max_tokens(self) -> int:
        return self._max_tokens

    def max_map_task_templates(self) -> int:
        return self._max_map_task_templates

    def update(self, req_slots, token_indices, cu_tokens, selection: Selection, stream=None) -> GqaReplayShape:
        if len(req_slots) != len(token_indices) or len(cu_tokens) != len(req_slots) + 1:
            raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "GQA batch arrays have inconsistent lengths")
        shape = GqaReplayShape()
        _lib.check(_lib.lib().khm_gqa_metadata_update(self._handle, _u32(req_slots), _u32(token_indices), _u32(cu_tokens),
                                                      len(req_slots), selection._handle,
                                                      ctypes.c_void_p(stream_handle(stream)), ctypes.byref(shape)))
        return shape

    def buffer(self, which: int) -> Buffer:
        out = Buffer()
        _lib.check(_lib.lib().khm_gqa_metadata_buffer(self._handle, which, ctypes.byref(out)))
        return out

    def host(self, which: int) -> np.ndarray:
        pointer = ctypes.POINTER(ctypes.c_uint32)()
        count = ctypes.c_uint64()
        _lib.check(_lib.lib().khm_gqa_metadata_host(self._handle, which, ctypes.byref(pointer), ctypes.byref(count)))
        return np.ctypeslib.as_array(pointer, shape=(count.value,)).copy()

    def req_slots(self):
        return self.buffer(REQ_SLOTS)

    def flat_token_indices(self):
        return self.buffer(FLAT_TOKEN_INDICES)

    def visible_kv_token_ranges(self):
        return self.buffer(VISIBLE_KV_TOKEN_RANGES)

    def q_token_ranges(self):
        return self.buffer(Q_TOKEN_RANGES)

    def sdpa_map_task_templates(self):
        return self.buffer(SDPA_MAP_TASK_TEMPLATES)

    def cu_sdpa_partial_outputs(self):
        return self.buffer(CU_SDPA_PARTIAL_OUTPUTS)
