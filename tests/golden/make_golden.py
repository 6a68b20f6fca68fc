#!/usr/bin/env python3
"""Writes the golden fixtures of this directory: inputs built exactly as the reference's component tests build theirs
(same generator, seeds, shapes, page tables and task templates) and the expected outputs from the CPU oracle.

    python tests/golden/make_golden.py        (from the repository root; needs the built oracle, no GPU)

Fixtures (numpy .npz, inputs as bit patterns, expected outputs as f32):
  paged_ranges_d{D}_p{tokens_per_page}_{bf16|fp8}.npz
      test_replay_paged_ranges (crates/inference-backend-metal/src/components/gqa/sdpa/sliced_q_test.rs:52-217):
      Hq6/Hkv2, two layers, two page ids per block, requests of 36 and 7 tokens in swapped slots, pages dealt from 11
      downwards, Q seed 17, K seed 31, V seed 47 (`generated_bf16_values`, sliced_q_test.rs:611-619), three Q ranges,
      six task templates, plain and windowed visible ranges.  The reference stores FP8 pages; the bf16 twin holds the
      same (FP8-representable) values in 16-bit pages.
  ragged_decode_d{D}.npz
      test_replay_ragged_two_requests-style decode (sliced_kv_test.rs:117-228 builds it at toy sizes; here at the kernel's
      head dims): two requests of 37 and 5 visible tokens, seeds 0x8B1D5A73..75 (`generated_values`,
      sliced_kv_test.rs:501-509), slices of 16 tokens.
The reference's Rust oracle is not run (no toolchain here); the oracle under oracle/ that produces the expected values is
pinned separately by tests/test_oracle.py.
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import gqa_oracle as oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
U32_MAX = 0xFFFFFFFF


def lcg(count: int, seed: int) -> np.ndarray:
    """(state >> 8) / 2^24 of the reference's linear congruential generator, as f32."""
    out = np.empty(count, dtype=np.float32)
    state = seed
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(state >> 8) / np.float32(16777216.0)
    return out


def generated_bf16_values(count: int, seed: int) -> np.ndarray:
    """sliced_q_test.rs:611-619."""
    return oracle.bf16_round(lcg(count, seed) - np.float32(0.5))


def generated_values(count: int, seed: int) -> np.ndarray:
    """sliced_kv_test.rs:501-509."""
    return lcg(count, seed) * np.float32(2.0) - np.float32(1.0)


def paged_ranges(head_dim: int, tpp: int, fp8: bool) -> dict:
    hq, hkv = 6, 2
    geom = oracle.Geometry(hq, hkv, head_dim, tpp, head_dim ** -0.5, 2, 3, 2, oracle.KV_FP8_E4M3FN if fp8 else oracle.KV_BF16)
    contexts = [36, 7]
    kv_width = hkv * head_dim
    keys = [oracle.fp8_round_trip(generated_bf16_values(n * kv_width, 31)).reshape(n, hkv, head_dim) for n in contexts]
    values = [oracle.fp8_round_trip(generated_bf16_values(n * kv_width, 47)).reshape(n, hkv, head_dim) for n in contexts]
    page_table = np.full((2, 2, 6), U32_MAX, dtype=np.uint32)
    page_lists, next_page = [], 11
    for req, slot in enumerate([1, 0]):
        pages = []
        for p in range(-(-contexts[req] // tpp)):
            page_table[slot, 1, p] = next_page
            pages.append(next_page)
            next_page -= 1
        page_lists.append(pages)
    kv_pages = oracle.pack_pages(geom, 12, list(zip(keys, values)), page_lists)
    q_bits = oracle.f32_to_bf16_bits(generated_bf16_values(20 * hq * head_dim, 17)).reshape(20, hq, head_dim)
    slots = np.ones(20, dtype=np.uint32)
    slots[17] = 0
    ranges = np.array([[0, 16], [16, 17], [17, 18], [U32_MAX, U32_MAX]], dtype=np.uint32)
    templates = np.array([[0, 0, 16], [0, 16, 35], [1, 0, 16], [1, 16, 36], [2, 0, 7], [2, 7, 7], [U32_MAX] * 3, [U32_MAX] * 3],
                         dtype=np.uint32)
    cu = np.array([0, 2, 4, 6, U32_MAX], dtype=np.uint32)
    out = dict(head_dim=head_dim, tokens_per_page=tpp, fp8=int(fp8), q_bits=q_bits, kv_pages=kv_pages, page_ids=page_table.reshape(-1),
               req_slots=slots, q_token_ranges=ranges, templates=templates, cu=cu)
    for name, windowed in (("plain", False), ("windowed", True)):
        visible = np.zeros((20, 2), dtype=np.uint32)
        for token in range(18):
            req = int(token == 17)
            end = 20 + token if req == 0 else 7
            begin = (end - 3 if req == 0 else end) if windowed else 0
            visible[token] = (begin, end)
        out[f"visible_{name}"] = visible
        out[f"expected_{name}"] = oracle.paged_gqa(geom, q_bits[:18], kv_pages, slots[:18], page_table.reshape(-1), visible[:18], layer=1)
    return out


def ragged_decode(head_dim: int) -> dict:
    hq, hkv, tpp = 8, 2, 16
    contexts = [37, 5]
    geom = oracle.Geometry(hq, hkv, head_dim, tpp, 0.5 * head_dim ** -0.5, 1, 3, 1)
    kv_width = hkv * head_dim
    keys = [oracle.bf16_round(generated_values(n * kv_width, 0x8B1D5A74 + 16 * r)).reshape(n, hkv, head_dim) for r, n in enumerate(contexts)]
    values = [oracle.bf16_round(generated_values(n * kv_width, 0x8B1D5A75 + 16 * r)).reshape(n, hkv, head_dim) for r, n in enumerate(contexts)]
    page_lists = [[4, 2, 0], [3]]
    page_table = np.full((2, 1, 3), U32_MAX, dtype=np.uint32)
    for r, pages in enumerate(page_lists):
        page_table[r, 0, :len(pages)] = pages
    kv_pages = oracle.pack_pages(geom, 5, list(zip(keys, values)), page_lists)
    q_bits = oracle.f32_to_bf16_bits(oracle.bf16_round(generated_values(2 * hq * head_dim, 0x8B1D5A73))).reshape(2, hq, head_dim)
    slots = np.array([0, 1], dtype=np.uint32)
    visible = np.array([[0, 37], [0, 5]], dtype=np.uint32)
    templates = np.array([[0, 0, 16], [0, 16, 32], [0, 32, 37], [1, 0, 5]], dtype=np.uint32)
    cu = np.array([0, 3, 4], dtype=np.uint32)
    expected = oracle.paged_gqa(geom, q_bits, kv_pages, slots, page_table.reshape(-1), visible)
    return dict(head_dim=head_dim, tokens_per_page=tpp, scale=np.float32(geom.scale), q_bits=q_bits, kv_pages=kv_pages,
                page_ids=page_table.reshape(-1), req_slots=slots, visible=visible, templates=templates, cu=cu, expected=expected)


def main() -> None:
    for head_dim, tpp, fp8 in [(128, 16, False), (128, 16, True), (256, 16, True), (256, 32, False)]:
        if True:
            name = f"paged_ranges_d{head_dim}_p{tpp}_{'fp8' if fp8 else 'bf16'}.npz"
            np.savez_compressed(os.path.join(HERE, name), **paged_ranges(head_dim, tpp, fp8))
            print(name)
    for head_dim in (128, 256):
        name = f"ragged_decode_d{head_dim}.npz"
        np.savez_compressed(os.path.join(HERE, name), **ragged_decode(head_dim))
        print(name)


if __name__ == "__main__":
    main()
