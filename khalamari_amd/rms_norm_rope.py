"""Mirror of `components::rms_norm_rope` (rms_norm_rope.rs:53-403): per-head RMSNorm, then default or Yarn rotary embedding."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, replace
from typing import Optional

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import DTYPE_BF16, DTYPE_F32, ReplayU32, RmsNormRopeBuffers, RmsNormRopeConfig, RopeScalingStruct


@dataclass(frozen=True)
class Yarn:
    """`RopeScaling::Yarn` (rms_norm_rope.rs:56-63)."""

    factor: float
    attention_factor: float
    beta_fast: float
    beta_slow: float
    original_max_position_embeddings: int
    truncate: bool


@dataclass(frozen=True)
class Config:
    """`rms_norm_rope::Config` (rms_norm_rope.rs:77-124); `rope_scaling` None is `RopeScaling::Default`."""

    num_heads: int
    head_dim: int
    rope_dim: int
    eps: float
    rope_theta: float
    rope_scaling: Optional[Yarn] = None
    dtype: int = DTYPE_BF16
    norm_weight_dtype: int = DTYPE_BF16

    @staticmethod
    def f32(num_heads, head_dim, rope_dim, eps, rope_theta) -> "Config":
        return Config(num_heads, head_dim, rope_dim, eps, rope_theta, None, DTYPE_F32, DTYPE_BF16)

    @staticmethod
    def bf16(num_heads, head_dim, rope_dim, eps, rope_theta) -> "Config":
        return Config(num_heads, head_dim, rope_dim, eps, rope_theta, None, DTYPE_BF16, DTYPE_BF16)

    def with_rope_scaling(self, rope_scaling: Optional[Yarn]) -> "Config":
        return replace(self, rope_scaling=rope_scaling)

    def with_norm_weight_dtype(self, dtype: int) -> "Config":
        return replace(self, norm_weight_dtype=dtype)

    def as_struct(self) -> RmsNormRopeConfig:
        y = self.rope_scaling
        scaling = RopeScalingStruct(0, 1.0, 1.0, 1.0, 1.0, 1, 0) if y is None else RopeScalingStruct(
            1, y.factor, y.attention_factor, y.beta_fast, y.beta_slow, y.original_max_position_embeddings, int(y.truncate))
        return RmsNormRopeConfig(self.num_heads, self.head_dim, self.rope_dim, self.eps, self.rope_theta, scaling, self.dtype,
                                 self.norm_weight_dtype)

    def yarn_correction_range(self):
        """`RopeScaling::yarn_kernel_parameters` (rms_norm_rope.rs:206-243): (correction_low, correction_high)."""
        config, low, high = self.as_struct(), ctypes.c_float(), ctypes.c_float()
        _lib.check(_lib.lib().khm_rms_norm_rope_yarn_correction_range(ctypes.byref(config), ctypes.byref(low), ctypes.byref(high)))
        return low.value, high.value

    def kernel_parameters(self):
        """`RopeScaling::kernel_parameters` (rms_norm_rope.rs:245-270): (inverse frequencies, attention factor)."""
        config, factor = self.as_struct(), ctypes.c_float()
        table = (ctypes.c_float * max(self.rope_dim // 2, 1))()
        _lib.check(_lib.lib().khm_rms_norm_rope_kernel_parameters(ctypes.byref(config), table, len(table), ctypes.byref(factor)))
        return list(table)[: self.rope_dim // 2], factor.value


@dataclass(frozen=True)
class Shape:
    """`rms_norm_rope::Shape` (rms_norm_rope.rs:272-284)."""

    num_total_tokens: int


class Compute:
    """`rms_norm_rope::Compute` (rms_norm_rope.rs:294-342): `invoke` validates and enqueues one launch."""

    def __init__(self, config: Config):
        self.config = config
        config.kernel_parameters()

    def invoke(self, shape: Shape, *, input, norm_weight, flat_token_indices, output, num_active_tokens: ReplayU32, replay_parameters=None,
               stream=None) -> None:
        config = self.config.as_struct()
        buffers = RmsNormRopeBuffers(view(input), view(norm_weight), view(flat_token_indices), view(output))
        _lib.check(_lib.lib().khm_rms_norm_rope(ctypes.byref(config), shape.num_total_tokens, ctypes.byref(buffers), num_active_tokens,
                                                param_block(replay_parameters), stream_handle(stream)))
