"""Mirror of `components::gqa::qgkv_split` (qgkv_split.rs:34-236): the gated projection row
`[Hq x (q head | gate head)][Hkv x k head][Hkv x v head]` of every active token goes to `q`, `g`, `k`, `v`."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import DTYPE_BF16, DTYPE_F32, ProjectionSplitConfig, ReplayU32


@dataclass(frozen=True)
class Config:
    """`qgkv_split::Config` (qgkv_split.rs:34-133)."""

    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    dtype: int

    GATED = True

    @classmethod
    def f32(cls, num_q_heads: int, num_kv_heads: int, head_dim: int):
        return cls(num_q_heads, num_kv_heads, head_dim, DTYPE_F32)

    @classmethod
    def bf16(cls, num_q_heads: int, num_kv_heads: int, head_dim: int):
        return cls(num_q_heads, num_kv_heads, head_dim, DTYPE_BF16)

    def c(self) -> ProjectionSplitConfig:
        return ProjectionSplitConfig(self.num_q_heads, self.num_kv_heads, self.head_dim, self.dtype)

    def item_size(self) -> int:
        return 4 if self.dtype == DTYPE_F32 else 2

    def projection_width(self) -> int:
        """`qgkv_width` (qgkv_split.rs:119-133): elements of one token's projection row."""
        c = self.c()
        width = _lib.lib().khm_gqa_qgkv_width(ctypes.byref(c)) if self.GATED else _lib.lib().khm_gqa_qkv_width(ctypes.byref(c))
        if width == 0:
            raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "GQA fused projection head count must fit u32")
        return int(width)

    def num_projection_slots(self, shape: "Shape") -> int:
        return shape.num_total_tokens * self.projection_width()

    def num_q_slots(self, shape: "Shape") -> int:
        return shape.num_total_tokens * self.num_q_heads * self.head_dim

    def num_kv_slots(self, shape: "Shape") -> int:
        return shape.num_total_tokens * self.num_kv_heads * self.head_dim

    def projection_bytes(self, shape: "Shape") -> int:
        return self.num_projection_slots(shape) * self.item_size()

    def q_bytes(self, shape: "Shape") -> int:
        return self.num_q_slots(shape) * self.item_size()

    def kv_bytes(self, shape: "Shape") -> int:
        return self.num_kv_slots(shape) * self.item_size()


@dataclass(frozen=True)
class Shape:
    """`qgkv_split::Shape` (qgkv_split.rs:136-147)."""

    num_total_tokens: int


class Compute:
    """`qgkv_split::Compute` (qgkv_split.rs:158-185); `invoke` enqueues on the stream."""

    def __init__(self, config: Config):
        self.config = config

    def invoke(self, shape: Shape, *, qgkv, q, g, k, v, num_active_tokens: ReplayU32, replay_parameters=None, stream=None) -> None:
        c = self.config.c()
        _lib.check(_lib.lib().khm_gqa_qgkv_split(ctypes.byref(c), shape.num_total_tokens, view(qgkv), view(q), view(g), view(k), view(v),
                                                 num_active_tokens, param_block(replay_parameters), stream_handle(stream)))
