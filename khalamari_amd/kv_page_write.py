"""Mirror of `components::gqa::kv_page_write` (kv_page_write.rs:60-283): bf16 K/V rows -> pages through the page table."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from ._buffers import param_block, stream_handle, view
from ._lib import DTYPE_BF16, DTYPE_FP8_E4M3FN, KvPageWriteBuffers, KvPageWriteConfig, KvPageWriteShape, PageTableLayoutStruct, ReplayU32


@dataclass(frozen=True)
class PageTableLayout:
    """`kv_page_write::PageTableLayout` (kv_page_write.rs:34-58)."""

    num_req_slots: int
    num_gqa_layers: int
    num_blocks: int
    num_page_ids_per_block: int

    def bytes(self) -> int:
        return self.num_req_slots * self.num_gqa_layers * self.num_blocks * self.num_page_ids_per_block * 4

    def as_struct(self) -> PageTableLayoutStruct:
        return PageTableLayoutStruct(self.num_req_slots, self.num_gqa_layers, self.num_blocks, self.num_page_ids_per_block)


@dataclass(frozen=True)
class Config:
    """`kv_page_write::Config` (kv_page_write.rs:60-66); `kv_dtype` picks FP8 E4M3FN pages (the reference) or bf16 pages."""

    num_kv_heads: int
    head_dim: int
    page_bytes: int
    dtype: int = DTYPE_BF16
    kv_dtype: int = DTYPE_FP8_E4M3FN

    def as_struct(self) -> KvPageWriteConfig:
        return KvPageWriteConfig(self.num_kv_heads, self.head_dim, self.page_bytes, self.dtype, self.kv_dtype)

    def num_tokens_per_page(self) -> int:
        config = self.as_struct()
        tokens = int(_lib.lib().khm_kv_page_write_num_tokens_per_page(ctypes.byref(config)))
        if tokens == 0:
            raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "GQA page_bytes must be divisible by the K/V bytes per token")
        return tokens

    def flat_kv_bytes(self, shape: "Shape") -> int:
        return shape.num_total_token_writes * self.num_kv_heads * self.head_dim * 2

    def index_bytes(self, shape: "Shape") -> int:
        return shape.num_total_token_writes * 4


@dataclass(frozen=True)
class Shape:
    """`kv_page_write::Shape` (kv_page_write.rs:115-134)."""

    num_total_token_writes: int
    page_table_layout: PageTableLayout

    def as_struct(self) -> KvPageWriteShape:
        return KvPageWriteShape(self.num_total_token_writes, self.page_table_layout.as_struct())

    def page_ids_bytes(self) -> int:
        return self.page_table_layout.bytes()


class Compute:
    """`kv_page_write::Compute` (kv_page_write.rs:147-183): `invoke` validates and enqueues one launch."""

    def __init__(self, config: Config):
        self.config = config
        config.num_tokens_per_page()

    def invoke(self, shape: Shape, *, pages, flat_k, flat_v, req_slots, flat_token_indices, page_ids, num_active_token_writes: ReplayU32,
               page_table_index: ReplayU32, replay_parameters=None, stream=None) -> None:
        config, cshape = self.config.as_struct(), shape.as_struct()
        buffers = KvPageWriteBuffers(view(pages), view(flat_k), view(flat_v), view(req_slots), view(flat_token_indices), view(page_ids))
        _lib.check(_lib.lib().khm_kv_page_write(ctypes.byref(config), ctypes.byref(cshape), ctypes.byref(buffers), num_active_token_writes,
                                                page_table_index, param_block(replay_parameters), stream_handle(stream)))


def fp8_decode_device(codes, bf16_out, count: int, stream=None) -> None:
    """E4M3FN codes -> bf16 on the device, as the Map kernels decode FP8 pages (gqa_fp8.metal:1-25)."""
    _lib.check(_lib.lib().khm_fp8_e4m3_to_bf16_device(view(codes), view(bf16_out), count, stream_handle(stream)))


def fp8_encode_device(bf16_in, codes, count: int, stream=None) -> None:
    """bf16 -> E4M3FN codes on the device, as the page writer encodes (gqa_kv_page_write.metal:5-31)."""
    _lib.check(_lib.lib().khm_bf16_to_fp8_e4m3_device(view(bf16_in), view(codes), count, stream_handle(stream)))
