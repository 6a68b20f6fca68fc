"""Mirror of `components::gqa::activation_gate` (activation_gate.rs:35-168): out = attention * sigmoid(gate)."""
from __future__ import annotations

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import ReplayU32


def invoke(dtype: int, num_q_heads: int, head_dim: int, num_total_tokens: int, attention_output, gates, output,
           num_active_tokens: ReplayU32, replay_parameters=None, stream=None) -> None:
    _lib.check(_lib.lib().khm_gqa_activation_gate(dtype, num_q_heads, head_dim, num_total_tokens, view(attention_output),
                                                  view(gates), view(output), num_active_tokens,
                                                  param_block(replay_parameters), stream_handle(stream)))
