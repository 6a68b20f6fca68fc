"""Mirror of `components::gqa::sdpa::sliced_kv` (sdpa/sliced_kv.rs): `Config`, `Shape`, `Scratch`, `Compute`."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import (DTYPE_BF16, GqaSdpaConfig, GqaSdpaShape, PageTableLayout, ReplayU32, SdpaVariant,
                   SlicedKvMapBuffers, SlicedKvReduceBuffers, SlicedKvStaticBuffers)


@dataclass(frozen=True)
class Layout:
    """`PageTableLayout` (components/gqa/kv_page_write.rs:34-58)."""

    num_req_slots: int = 1
    num_gqa_layers: int = 1
    num_blocks: int = 1
    num_page_ids_per_block: int = 1

    def c(self) -> PageTableLayout:
        return PageTableLayout(self.num_req_slots, self.num_gqa_layers, self.num_blocks, self.num_page_ids_per_block)


@dataclass(frozen=True)
class Config:
    """`sliced_kv::Config` (sliced_kv.rs:91-99) plus the explicit K/V and partial dtypes."""

    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    page_bytes: int
    page_table_layout: Layout = field(default_factory=Layout)
    dtype: int = DTYPE_BF16
    kv_dtype: int = DTYPE_BF16
    partial_dtype: int = DTYPE_BF16

    def c(self) -> GqaSdpaConfig:
        return GqaSdpaConfig(self.num_q_heads, self.num_kv_heads, self.head_dim, self.scale, self.page_bytes,
                             self.page_table_layout.c(), self.dtype, self.kv_dtype, self.partial_dtype)

    def num_tokens_per_page(self) -> int:
        c = self.c()
        return int(_lib.lib().khm_gqa_sdpa_num_tokens_per_page(ctypes.byref(c)))

    def q_heads_per_kv_head(self) -> int:
        return self.num_q_heads // self.num_kv_heads

    def sdpa_config(self):
        from .sdpa import Config as SdpaConfig

        return SdpaConfig(self.dtype, self.num_q_heads, self.num_kv_heads, self.head_dim, self.num_tokens_per_page())

    def q_bytes(self, shape: "Shape") -> int:
        c, s = self.c(), shape.c()
        return int(_lib.lib().khm_gqa_sdpa_q_bytes(ctypes.byref(c), ctypes.byref(s)))

    def page_ids_bytes(self) -> int:
        c = self.c()
        return int(_lib.lib().khm_gqa_sdpa_page_ids_bytes(ctypes.byref(c)))

    def partial_output_stats_bytes(self, shape: "Shape") -> int:
        c, s = self.c(), shape.c()
        return int(_lib.lib().khm_sliced_kv_partial_output_stats_bytes(ctypes.byref(c), ctypes.byref(s)))

    def partial_output_bytes(self, shape: "Shape") -> int:
        c, s = self.c(), shape.c()
        return int(_lib.lib().khm_sliced_kv_partial_output_bytes(ctypes.byref(c), ctypes.byref(s)))

    def num_output_values(self, shape: "Shape") -> int:
        return shape.num_total_tokens * self.num_q_heads * self.head_dim


@dataclass(frozen=True)
class Shape:
    """`sliced_kv::Shape` (sliced_kv.rs:215-219)."""

    num_total_tokens: int
    num_total_sdpa_map_task_templates: int

    def c(self) -> GqaSdpaShape:
        return GqaSdpaShape(self.num_total_tokens, 0, self.num_total_sdpa_map_task_templates)


class Scratch:
    """`sliced_kv::Scratch` (sliced_kv.rs:265-320): partial sums / maxima / outputs, zero-initialised."""

    def __init__(self, device, config: Config, shape: Shape):
        import torch

        self.partial_exp_sums = torch.zeros(config.partial_output_stats_bytes(shape), dtype=torch.uint8, device=device)
        self.partial_max_logits = torch.zeros(config.partial_output_stats_bytes(shape), dtype=torch.uint8, device=device)
        self.partial_output = torch.zeros(config.partial_output_bytes(shape), dtype=torch.uint8, device=device)


class Compute:
    """`sliced_kv::Compute` (sliced_kv.rs:315-388): `invoke_map` / `invoke_reduce` enqueue on a stream."""

    def __init__(self, config: Config, execution: SdpaVariant, shape: Shape):
        self.config, self.execution, self.shape = config, execution, shape
        handle = ctypes.c_void_p()
        c, s = config.c(), shape.c()
        _lib.check(_lib.lib().khm_sliced_kv_create(ctypes.byref(c), ctypes.byref(execution), ctypes.byref(s),
                                                   ctypes.byref(handle)))
        self._handle = handle

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None and getattr(_lib, "_lib", None) is not None:
            _lib._lib.khm_sliced_kv_destroy(handle)
            self._handle = None

    def map_kernel_id(self) -> int:
        return int(_lib.lib().khm_sliced_kv_map_kernel_id(self._handle))

    def reduce_kernel_id(self) -> int:
        return int(_lib.lib().khm_sliced_kv_reduce_kernel_id(self._handle))

    def invoke_map(self, *, q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, partial_exp_sums,
                   partial_max_logits, partial_output, page_table_index: ReplayU32, num_active_tokens: ReplayU32,
                   num_active_kv_splits: ReplayU32, replay_parameters=None, stream=None) -> None:
        buffers = SlicedKvMapBuffers(view(q), view(kv_pages), view(req_slots), view(page_ids),
                                     view(sdpa_map_task_templates), view(partial_exp_sums), view(partial_max_logits),
                                     view(partial_output))
        _lib.check(_lib.lib().khm_sliced_kv_map(self._handle, ctypes.byref(buffers), page_table_index, num_active_tokens,
                                                num_active_kv_splits, param_block(replay_parameters),
                                                stream_handle(stream)))

    def arrival_counters_bytes(self) -> int:
        c, s = self.config.c(), self.shape.c()
        return int(_lib.lib().khm_sliced_kv_arrival_counters_bytes(ctypes.byref(c), ctypes.byref(self.execution), ctypes.byref(s)))

    def invoke_map_reduce(self, *, q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, partial_exp_sums,
                          partial_max_logits, partial_output, cu_sdpa_partial_outputs, output, arrival_counters,
                          page_table_index: ReplayU32, num_active_tokens: ReplayU32, num_active_kv_splits: ReplayU32,
                          gates=None, replay_parameters=None, stream=None) -> None:
        """Map and Reduce (optionally gated) in one launch; `arrival_counters` must start zeroed."""
        map_buffers = SlicedKvMapBuffers(view(q), view(kv_pages), view(req_slots), view(page_ids),
                                         view(sdpa_map_task_templates), view(partial_exp_sums), view(partial_max_logits),
                                         view(partial_output))
        reduce_buffers = SlicedKvReduceBuffers(view(partial_exp_sums), view(partial_max_logits), view(partial_output),
                                               view(cu_sdpa_partial_outputs), view(output))
        gate_view = view(gates) if gates is not None else _lib.Buffer(None, 0)
        _lib.check(_lib.lib().khm_sliced_kv_map_reduce(self._handle, ctypes.byref(map_buffers), ctypes.byref(reduce_buffers),
                                                       gate_view, view(arrival_counters), page_table_index, num_active_tokens,
                                                       num_active_kv_splits, param_block(replay_parameters),
                                                       stream_handle(stream)))

    def invoke_map_reduce_static(self, *, q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, cu_sdpa_partial_outputs,
                                 output, page_table_index: ReplayU32, num_active_tokens: ReplayU32,
                                 num_active_kv_splits: ReplayU32, gates=None, replay_parameters=None, stream=None) -> None:
        """`invoke_map_reduce` with the partial states and arrival counters in the library's own static device array:
        nothing is allocated and no workspace is passed (no counterpart in the reference)."""
        buffers = SlicedKvStaticBuffers(view(q), view(kv_pages), view(req_slots), view(page_ids), view(sdpa_map_task_templates),
                                        view(cu_sdpa_partial_outputs), view(output))
        gate_view = view(gates) if gates is not None else _lib.Buffer(None, 0)
        _lib.check(_lib.lib().khm_sliced_kv_map_reduce_static(self._handle, ctypes.byref(buffers), gate_view, page_table_index,
                                                              num_active_tokens, num_active_kv_splits,
                                                              param_block(replay_parameters), stream_handle(stream)))

    def invoke_reduce(self, *, partial_exp_sums, partial_max_logits, partial_output, cu_sdpa_partial_outputs, output,
                      num_active_tokens: ReplayU32, gates=None, replay_parameters=None, stream=None) -> None:
        buffers = SlicedKvReduceBuffers(view(partial_exp_sums), view(partial_max_logits), view(partial_output),
                                        view(cu_sdpa_partial_outputs), view(output))
        if gates is None:
            _lib.check(_lib.lib().khm_sliced_kv_reduce(self._handle, ctypes.byref(buffers), num_active_tokens,
                                                       param_block(replay_parameters), stream_handle(stream)))
        else:
            _lib.check(_lib.lib().khm_sliced_kv_reduce_gated(self._handle, ctypes.byref(buffers), view(gates),
                                                             num_active_tokens, param_block(replay_parameters),
                                                             stream_handle(stream)))
