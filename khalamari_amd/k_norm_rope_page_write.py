"""K RMSNorm + RoPE fused with the K/V page write: the three recordings `k_norm_rope -> scratch.k_norm_rope -> kv_page_write`
of `GQA::record` (crates/inference-executor-metal/src/attn/gqa/backend.rs:382-412) as one launch."""
from __future__ import annotations

import ctypes

from . import _lib, kv_page_write, rms_norm_rope
from ._buffers import param_block, stream_handle, view
from ._lib import KNormRopePageWriteBuffers, ReplayU32


class Compute:
    """Pairs an `rms_norm_rope::Config` over the KV heads with a `kv_page_write::Config`; `invoke` validates both and
    enqueues one launch that leaves in the pages exactly what the two components would have written."""

    def __init__(self, norm_config: rms_norm_rope.Config, page_config: kv_page_write.Config):
        self.norm_config, self.page_config = norm_config, page_config
        norm_config.kernel_parameters()
        page_config.num_tokens_per_page()

    def invoke(self, shape: kv_page_write.Shape, *, pages, k, v, norm_weight, req_slots, flat_token_indices, page_ids,
               num_active_tokens: ReplayU32, page_table_index: ReplayU32, replay_parameters=None, stream=None) -> None:
        norm, page, cshape = self.norm_config.as_struct(), self.page_config.as_struct(), shape.as_struct()
        buffers = KNormRopePageWriteBuffers(view(pages), view(k), view(v), view(norm_weight), view(req_slots), view(flat_token_indices),
                                            view(page_ids))
        _lib.check(_lib.lib().khm_k_norm_rope_page_write(ctypes.byref(norm), ctypes.byref(page), ctypes.byref(cshape), ctypes.byref(buffers),
                                                         num_active_tokens, page_table_index, param_block(replay_parameters),
                                                         stream_handle(stream)))
