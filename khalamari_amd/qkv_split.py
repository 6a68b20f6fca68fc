"""Mirror of `components::gqa::qkv_split` (qkv_split.rs:35-233): the ungated projection row
`[Hq x q head][Hkv x k head][Hkv x v head]` of every active token goes to `q`, `k`, `v`."""
from __future__ import annotations

import ctypes

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import ReplayU32
from .qgkv_split import Config as _GatedConfig
from .qgkv_split import Shape  # noqa: F401


class Config(_GatedConfig):
    """`qkv_split::Config` (qkv_split.rs:35-131): the same fields; `projection_width` is `qkv_width`."""

    GATED = False


class Compute:
    """`qkv_split::Compute` (qkv_split.rs:153-194)."""

    def __init__(self, config: Config):
        self.config = config

    def invoke(self, shape: Shape, *, qkv, q, k, v, num_active_tokens: ReplayU32, replay_parameters=None, stream=None) -> None:
        c = self.config.c()
        _lib.check(_lib.lib().khm_gqa_qkv_split(ctypes.byref(c), shape.num_total_tokens, view(qkv), view(q), view(k), view(v),
                                                num_active_tokens, param_block(replay_parameters), stream_handle(stream)))
