"""MI355X (gfx950) paged GQA split-KV SDPA component behind a C ABI.

The package is a thin host-side mirror of the reference's backend component interface
(`components::gqa::sdpa::{sliced_kv, sliced_q}`, `components::gqa::activation_gate`) and of the
executor-side selector and metadata (`attn::gqa::{sdpa, batch_metadata}`); all arithmetic and all
host logic live in `lib/libkhm_gqa_sdpa.so` (sources under `csrc/`, ABI in `include/khm_gqa_sdpa.h`).
"""
from . import _lib  # noqa: F401

__all__ = ["_lib", "sdpa", "sliced_kv", "sliced_q", "activation_gate", "qgkv_split", "qkv_split", "kv_page_write", "bidi_block_sdpa", "bidi_block_metadata", "rms_norm_rope", "k_norm_rope_page_write", "projection_norm_rope_page_write", "selector", "batch_metadata", "replay"]
