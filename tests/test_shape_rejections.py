"""The shape domains the reference rejects with a panic are rejected here with the same message, before any device call
(sliced_kv_test.rs:44-55, sliced_q_test.rs:403-433, activation_gate.rs:252-260, kv_page_write.rs:263-283).  CPU only."""
import ctypes

import pytest

from khalamari_amd import _lib, kv_page_write as kpw, sdpa, sliced_kv, sliced_q
from khalamari_amd._lib import DTYPE_BF16, Buffer, KhmError, ReplayU32

U32_MAX = 0xFFFFFFFF


def _sliced_q_config(head_dim, tokens_per_page):
    """`sliced_q_workload(head_dim, tokens_per_page)` of sliced_q_test.rs:435-458: 5 Q heads over 1 KV head (bf16 pages here)."""
    return sliced_q.Config(5, 1, head_dim, 0.1, 2 * tokens_per_page * head_dim * 2)


def _per_head_variant(head_dim, tokens_per_page):
    return sdpa.ExecutionVariant.sliced_q_per_head(sdpa.Config(DTYPE_BF16, 5, 1, head_dim, tokens_per_page), 8, 16, 5)


def test_sdpa_shape_rejects_shader_count_overflow():
    config = sliced_kv.Config(8, 2, 128, 0.1, 2 * 2 * 16 * 128 * 2)
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), 128, 128, 4)
    with pytest.raises(KhmError, match="GQA SDPA query/output exceeds the shader u32 count domain"):
        sliced_kv.Compute(config, variant, sliced_kv.Shape(1 << 30, 1))


def test_sliced_q_shape_rejects_unsupported_profile():
    with pytest.raises(KhmError, match="GQA SplitKV SlicedQ supports only"):
        sliced_q.Compute.new(_sliced_q_config(192, 8), _per_head_variant(128, 8), sliced_q.Shape(8, 1, 1))


def test_sliced_q_shape_rejects_shader_index_overflow():
    with pytest.raises(KhmError, match="GQA SplitKV SlicedQ Q-token-range metadata exceeds the shader u32 element-index domain"):
        sliced_q.Compute.new(_sliced_q_config(256, 16), _per_head_variant(256, 16), sliced_q.Shape(U32_MAX, U32_MAX, U32_MAX))


def test_sliced_q_shape_rejects_visible_range_index_overflow():
    with pytest.raises(KhmError, match="GQA SplitKV SlicedQ visible K/V-token-range metadata exceeds the shader u32 element-index domain"):
        sliced_q.Compute.new(_sliced_q_config(256, 16), _per_head_variant(256, 16), sliced_q.Shape(U32_MAX, 1, 1))


def test_activation_gate_shape_rejects_shader_count_overflow():
    empty = Buffer(0, 0)
    with pytest.raises(KhmError, match="GQA activation/gate exceeds the shader u32 count domain"):
        _lib.check(_lib.lib().khm_gqa_activation_gate(DTYPE_BF16, 2, 2, 1 << 30, empty, empty, empty, ReplayU32.fixed(1), None, None))


def test_kv_page_write_shape_rejects_shader_count_overflow():
    config = kpw.Config(2, 2, 16).as_struct()
    shape = kpw.Shape(1 << 30, kpw.PageTableLayout(1, 1, 1, 1)).as_struct()
    buffers = _lib.KvPageWriteBuffers()
    with pytest.raises(KhmError, match="GQA KV page-write threads exceeds the shader u32 count domain"):
        _lib.check(_lib.lib().khm_kv_page_write(ctypes.byref(config), ctypes.byref(shape), ctypes.byref(buffers), ReplayU32.fixed(1),
                                                ReplayU32.fixed(0), None, None))
