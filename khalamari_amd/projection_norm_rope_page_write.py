"""The projection split, Q RMSNorm + RoPE, K RMSNorm + RoPE and the K/V page write as one launch: the recordings
`qgkv_to_q_g_k_v -> q_norm_rope -> k_norm_rope -> kv_page_write` of `GQA::record`
(crates/inference-executor-metal/src/attn/gqa/backend.rs:358-412)."""
from __future__ import annotations

import ctypes

from . import _lib, kv_page_write, rms_norm_rope
from ._buffers import param_block, stream_handle, view
from ._lib import Buffer, ProjectionNormRopePageWriteBuffers, ReplayU32


class Compute:
    """Pairs the Q and K `rms_norm_rope::Config`s with a `kv_page_write::Config`; `invoke` enqueues one launch that leaves in
    `q_output`, `gate_output` and the pages exactly what the split, the Q norm + RoPE and the fused K writer would."""

    def __init__(self, q_norm_config: rms_norm_rope.Config, k_norm_config: rms_norm_rope.Config, page_config: kv_page_write.Config,
                 gated: bool = True):
        self.q_norm_config, self.k_norm_config, self.page_config, self.gated = q_norm_config, k_norm_config, page_config, gated
        q_norm_config.kernel_parameters()
        k_norm_config.kernel_parameters()
        page_config.num_tokens_per_page()

    def projection_width(self) -> int:
        """Elements of one token's projection row (`qgkv_width` / `qkv_width`, qgkv_split.rs:119-133)."""
        q, k = self.q_norm_config, self.k_norm_config
        return ((2 if self.gated else 1) * q.num_heads + 2 * k.num_heads) * q.head_dim

    def invoke(self, shape: kv_page_write.Shape, *, projection, q_norm_weight, k_norm_weight, q_output, pages, req_slots, flat_token_indices,
               page_ids, num_active_tokens: ReplayU32, page_table_index: ReplayU32, gate_output=None, replay_parameters=None,
               stream=None) -> None:
        q_norm, k_norm = self.q_norm_config.as_struct(), self.k_norm_config.as_struct()
        page, cshape = self.page_config.as_struct(), shape.as_struct()
        buffers = ProjectionNormRopePageWriteBuffers(view(projection), view(q_norm_weight), view(k_norm_weight), view(q_output),
                                                     view(gate_output) if gate_output is not None else Buffer(0, 0), view(pages),
                                                     view(req_slots), view(flat_token_indices), view(page_ids))
        _lib.check(_lib.lib().khm_gqa_projection_norm_rope_page_write(
            1 if self.gated else 0, ctypes.byref(q_norm), ctypes.byref(k_norm), ctypes.byref(page), ctypes.byref(cshape), ctypes.byref(buffers),
            num_active_tokens, page_table_index, param_block(replay_parameters), stream_handle(stream)))
