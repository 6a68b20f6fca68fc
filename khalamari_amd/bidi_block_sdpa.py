"""Mirror of `components::gqa::bidi_block_sdpa` (bidi_block_sdpa.rs:44-340): dense bidirectional attention over a
request block, written as the last partial state of each Q range in the split-KV partial layout."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import DTYPE_BF16, DTYPE_F32, BidiBlockSdpaBuffers, BidiBlockSdpaConfig, BidiBlockSdpaShape, ReplayU32


@dataclass(frozen=True)
class Config:
    """`bidi_block_sdpa::Config` (bidi_block_sdpa.rs:55-63)."""

    block_size: int
    max_q_tokens: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    dtype: int = DTYPE_BF16

    def item_size(self) -> int:
        return 4 if self.dtype == DTYPE_F32 else 2

    def partial_output_stat_elements(self, shape: "Shape") -> int:
        return shape.num_total_partial_output_slots * self.num_q_heads * self.max_q_tokens

    def partial_output_values(self, shape: "Shape") -> int:
        return self.partial_output_stat_elements(shape) * self.head_dim

    def as_struct(self) -> BidiBlockSdpaConfig:
        return BidiBlockSdpaConfig(self.block_size, self.max_q_tokens, self.num_q_heads, self.num_kv_heads, self.head_dim, self.scale, self.dtype)


@dataclass(frozen=True)
class Shape:
    """`bidi_block_sdpa::Shape` (bidi_block_sdpa.rs:140-145)."""

    num_total_tokens: int
    num_total_q_token_ranges: int
    num_total_partial_output_slots: int

    def as_struct(self) -> BidiBlockSdpaShape:
        return BidiBlockSdpaShape(self.num_total_tokens, self.num_total_q_token_ranges, self.num_total_partial_output_slots)


class Compute:
    """`bidi_block_sdpa::Compute` (bidi_block_sdpa.rs:187-245): `invoke` validates and enqueues one launch."""

    def __init__(self, config: Config):
        self.config = config

    def invoke(self, shape: Shape, num_active_q_token_ranges: ReplayU32, *, q, local_k, local_v, q_token_ranges, cu_sdpa_partial_outputs,
               partial_exp_sums, partial_max_logits, partial_output, replay_parameters=None, stream=None) -> None:
        config, cshape = self.config.as_struct(), shape.as_struct()
        buffers = BidiBlockSdpaBuffers(view(q), view(local_k), view(local_v), view(q_token_ranges), view(cu_sdpa_partial_outputs),
                                       view(partial_exp_sums), view(partial_max_logits), view(partial_output))
        _lib.check(_lib.lib().khm_bidi_block_sdpa(ctypes.byref(config), ctypes.byref(cshape), ctypes.byref(buffers), num_active_q_token_ranges,
                                                  param_block(replay_parameters), stream_handle(stream)))
