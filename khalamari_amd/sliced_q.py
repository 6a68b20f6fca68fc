"""Mirror of `components::gqa::sdpa::sliced_q` (sdpa/sliced_q.rs): `Config`, `Shape`, `Compute` (+ direct output)."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import (GqaSdpaShape, ReplayU32, SdpaVariant, SlicedQDirectBuffers, SlicedQMapBuffers, SlicedQReduceBuffers)
from .sliced_kv import Config as _BaseConfig
from .sliced_kv import Layout  # noqa: F401


class Config(_BaseConfig):
    """`sliced_q::Config` (sliced_q.rs:171-179); same fields as the sliced-KV config."""

    def partial_output_bytes(self, execution: SdpaVariant, shape: "Shape") -> int:  # type: ignore[override]
        c, s = self.c(), shape.c()
        return int(_lib.lib().khm_sliced_q_partial_output_bytes(ctypes.byref(c), ctypes.byref(execution), ctypes.byref(s)))

    def partial_output_stats_bytes(self, execution: SdpaVariant, shape: "Shape") -> int:  # type: ignore[override]
        c, s = self.c(), shape.c()
        return int(_lib.lib().khm_sliced_q_partial_output_stats_bytes(ctypes.byref(c), ctypes.byref(execution),
                                                                      ctypes.byref(s)))


@dataclass(frozen=True)
class Shape:
    """`sliced_q::Shape` (sliced_q.rs:248-253)."""

    num_total_tokens: int
    num_total_q_token_tiles: int
    num_total_sdpa_map_task_templates: int

    def c(self) -> GqaSdpaShape:
        return GqaSdpaShape(self.num_total_tokens, self.num_total_q_token_tiles, self.num_total_sdpa_map_task_templates)


class Compute:
    """`sliced_q::Compute` (sliced_q.rs:323-504): `new` / `new_direct`, `invoke_map`, `invoke_direct`, `invoke_reduce`."""

    def __init__(self, config: Config, execution: SdpaVariant, shape: Shape, direct: bool = False):
        self.config, self.execution, self.shape, self.direct = config, execution, shape, direct
        handle = ctypes.c_void_p()
        c, s = config.c(), shape.c()
        _lib.check(_lib.lib().khm_sliced_q_create(ctypes.byref(c), ctypes.byref(execution), ctypes.byref(s),
                                                  1 if direct else 0, ctypes.byref(handle)))
        self._handle = handle

    @staticmethod
    def new(config: Config, execution: SdpaVariant, shape: Shape) -> "Compute":
        return Compute(config, execution, shape, direct=False)

    @staticmethod
    def new_direct(config: Config, execution: SdpaVariant, shape: Shape) -> "Compute":
        return Compute(config, execution, shape, direct=True)

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None and getattr(_lib, "_lib", None) is not None:
            _lib._lib.khm_sliced_q_destroy(handle)
            self._handle = None

    def map_kernel_id(self) -> int:
        return int(_lib.lib().khm_sliced_q_map_kernel_id(self._handle))

    def invoke_map(self, *, q, kv_pages, req_slots, page_ids, visible_kv_token_ranges, q_token_ranges,
                   sdpa_map_task_templates, partial_output, partial_exp_sums, partial_max_logits,
                   page_table_index: ReplayU32, num_active_tokens: ReplayU32, num_active_q_token_tiles: ReplayU32,
                   num_active_kv_splits: ReplayU32, replay_parameters=None, stream=None) -> None:
        buffers = SlicedQMapBuffers(view(q), view(kv_pages), view(req_slots), view(page_ids),
                                    view(visible_kv_token_ranges), view(q_token_ranges), view(sdpa_map_task_templates),
                                    view(partial_output), view(partial_exp_sums), view(partial_max_logits))
        _lib.check(_lib.lib().khm_sliced_q_map(self._handle, ctypes.byref(buffers), page_table_index, num_active_tokens,
                                               num_active_q_token_tiles, num_active_kv_splits,
                                               param_block(replay_parameters), stream_handle(stream)))

    def arrival_counters_bytes(self) -> int:
        c, s = self.config.c(), self.shape.c()
        return int(_lib.lib().khm_sliced_q_arrival_counters_bytes(ctypes.byref(c), ctypes.byref(self.execution), ctypes.byref(s)))

    def invoke_map_reduce(self, *, q, kv_pages, req_slots, page_ids, visible_kv_token_ranges, q_token_ranges,
                          sdpa_map_task_templates, partial_output, partial_exp_sums, partial_max_logits,
                          cu_sdpa_partial_outputs, output, arrival_counters, page_table_index: ReplayU32,
                          num_active_tokens: ReplayU32, num_active_q_token_tiles: ReplayU32, num_active_kv_splits: ReplayU32,
                          replay_parameters=None, stream=None) -> None:
        """Map and Reduce in one launch; `arrival_counters` must start zeroed."""
        map_buffers = SlicedQMapBuffers(view(q), view(kv_pages), view(req_slots), view(page_ids),
                                        view(visible_kv_token_ranges), view(q_token_ranges), view(sdpa_map_task_templates),
                                        view(partial_output), view(partial_exp_sums), view(partial_max_logits))
        reduce_buffers = SlicedQReduceBuffers(view(partial_output), view(partial_exp_sums), view(partial_max_logits),
                                              view(q_token_ranges), view(cu_sdpa_partial_outputs), view(output))
        _lib.check(_lib.lib().khm_sliced_q_map_reduce(self._handle, ctypes.byref(map_buffers), ctypes.byref(reduce_buffers),
                                                      view(arrival_counters), page_table_index, num_active_tokens,
                                                      num_active_q_token_tiles, num_active_kv_splits,
                                                      param_block(replay_parameters), stream_handle(stream)))

    def invoke_direct(self, *, q, kv_pages, req_slots, page_ids, visible_kv_token_ranges, q_token_ranges,
                      sdpa_map_task_templates, output, page_table_index: ReplayU32, num_active_tokens: ReplayU32,
                      num_active_q_token_tiles: ReplayU32, replay_parameters=None, stream=None, gates=None) -> None:
        """`gates` (bf16 [T][Hq][D]) fuses the sigmoid gate that follows the SDPA into the output write."""
        buffers = SlicedQDirectBuffers(view(q), view(kv_pages), view(req_slots), view(page_ids),
                                       view(visible_kv_token_ranges), view(q_token_ranges),
                                       view(sdpa_map_task_templates), view(output))
        if gates is not None:
            _lib.check(_lib.lib().khm_sliced_q_direct_gated(self._handle, ctypes.byref(buffers), view(gates), page_table_index,
                                                            num_active_tokens, num_active_q_token_tiles,
                                                            param_block(replay_parameters), stream_handle(stream)))
            return
        _lib.check(_lib.lib().khm_sliced_q_direct(self._handle, ctypes.byref(buffers), page_table_index,
                                                  num_active_tokens, num_active_q_token_tiles,
                                                  param_block(replay_parameters), stream_handle(stream)))

    def invoke_reduce(self, *, partial_output, partial_exp_sums, partial_max_logits, q_token_ranges,
                      cu_sdpa_partial_outputs, output, num_active_q_token_tiles: ReplayU32, replay_parameters=None,
                      stream=None, gates=None) -> None:
        buffers = SlicedQReduceBuffers(view(partial_output), view(partial_exp_sums), view(partial_max_logits),
                                       view(q_token_ranges), view(cu_sdpa_partial_outputs), view(output))
        if gates is not None:
            _lib.check(_lib.lib().khm_sliced_q_reduce_gated(self._handle, ctypes.byref(buffers), view(gates), num_active_q_token_tiles,
                                                            param_block(replay_parameters), stream_handle(stream)))
            return
        _lib.check(_lib.lib().khm_sliced_q_reduce(self._handle, ctypes.byref(buffers), num_active_q_token_tiles,
                                                  param_block(replay_parameters), stream_handle(stream)))
