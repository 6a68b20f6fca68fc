"""Workload builders shared by the parity tests: synthetic paged KV caches, fixed-slice map plans,
and the tolerance gate.  Expected values always come from the CPU oracle under `oracle/`."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from oracle import gqa_oracle as oracle

U32_MAX = 0xFFFFFFFF


@dataclass
class Workload:
    geom: oracle.Geometry
    q_bits: np.ndarray          # uint16 [T, Hq, D]
    kv_pages: np.ndarray        # uint8 [P, page_bytes]
    page_ids: np.ndarray        # uint32 [R, L, NB, PPB] flattened
    req_slots: np.ndarray       # uint32 [T]
    visible: np.ndarray         # uint32 [T, 2]
    cu_tokens: np.ndarray       # uint32 [R + 1]
    token_indices: np.ndarray   # uint32 [R] (history length per request)
    num_req_slots: int
    layer: int = 0

    @property
    def num_tokens(self) -> int:
        return int(self.req_slots.size)


def make_workload(*, num_q_heads, num_kv_heads, head_dim, tokens_per_page, histories, q_lens, seed, scale=None,
                  num_layers=1, layer=0, page_ids_per_block=1, permute=True, spare_pages=3, value_scale=1.0,
                  garbage_bits=None, req_slot_order=None, fp8_pages=False, key_drift=None) -> Workload:
    """Sequences r = 0..R-1 with `histories[r]` cached tokens and `q_lens[r]` new Q tokens (already in the cache).

    K/V/Q ~ N(0, value_scale) rounded to bf16.  Pages come from one shared pool, randomly permuted.
    `garbage_bits`, when given, fills every unused page slot (tokens past a sequence's end) with that bf16
    pattern, e.g. 0x7fc0 (NaN), to prove masked slots never reach the output (an FP8 code with `fp8_pages`).
    `key_drift` adds `key_drift * position` to dimension 0 of every key and sets dimension 0 of every query to 4: all
    scores of a sequence rise steadily along the context, so they keep outgrowing whatever running maximum an online
    softmax holds (its rescaling path runs many times) while the weights stay spread over many recent keys.
    `fp8_pages` stores K/V as FP8 E4M3FN codes; the values are quantised first, as the reference's tests do
    before their oracle sees them (sliced_kv_test.rs:484-493).
    """
    rng = np.random.default_rng(seed)
    R = len(histories)
    contexts = [int(h) + int(n) for h, n in zip(histories, q_lens)]
    pages_per_seq = [(c + tokens_per_page - 1) // tokens_per_page for c in contexts]
    max_pages = max(max(pages_per_seq), 1)
    num_blocks = (max_pages + page_ids_per_block - 1) // page_ids_per_block
    total_pages = sum(pages_per_seq) + spare_pages
    order = rng.permutation(total_pages) if permute else np.arange(total_pages)
    slots = list(req_slot_order) if req_slot_order is not None else list(range(R))
    num_req_slots = max(slots) + 1
    geom = oracle.Geometry(num_q_heads, num_kv_heads, head_dim, tokens_per_page,
                           float(scale if scale is not None else head_dim ** -0.5), num_layers, num_blocks,
                           page_ids_per_block, oracle.KV_FP8_E4M3FN if fp8_pages else oracle.KV_BF16)
    table = np.full((num_req_slots, num_layers, num_blocks * page_ids_per_block), U32_MAX, dtype=np.uint32)
    sequences, page_lists = [], []
    cursor = 0
    for r in range(R):
        ctx = contexts[r]
        k = rng.standard_normal((ctx, num_kv_heads, head_dim), dtype=np.float32) * value_scale
        if key_drift is not None:
            k[:, :, 0] += np.float32(key_drift) * np.arange(ctx, dtype=np.float32)[:, None]
        k = oracle.bf16_round(k)
        v = oracle.bf16_round(rng.standard_normal((ctx, num_kv_heads, head_dim), dtype=np.float32) * value_scale)
        if fp8_pages:
            k, v = oracle.fp8_round_trip(k), oracle.fp8_round_trip(v)
        pages = order[cursor:cursor + pages_per_seq[r]]
        cursor += pages_per_seq[r]
        table[slots[r], layer, :pages_per_seq[r]] = pages
        sequences.append((k, v))
        page_lists.append(pages)
    kv_pages = oracle.pack_pages(geom, total_pages, sequences, page_lists,
                                 fill_bits=0 if garbage_bits is None else garbage_bits)
    T = int(sum(q_lens))
    q = rng.standard_normal((T, num_q_heads, head_dim), dtype=np.float32) * value_scale
    if key_drift is not None:
        q[:, :, 0] = 4.0
    q_bits = oracle.f32_to_bf16_bits(q)
    req_slots = np.concatenate([np.full(n, slots[r], dtype=np.uint32) for r, n in enumerate(q_lens)])
    visible = np.zeros((T, 2), dtype=np.uint32)
    cu = np.zeros(R + 1, dtype=np.uint32)
    t = 0
    for r in range(R):
        for i in range(q_lens[r]):
            visible[t] = (0, histories[r] + i + 1)
            t += 1
        cu[r + 1] = t
    return Workload(geom, q_bits, kv_pages, table.reshape(-1), req_slots, visible, cu,
                    np.asarray(histories, dtype=np.uint32), num_req_slots, layer)


def fixed_slice_plan(histories, q_lens, max_q_tokens, kv_slice):
    """Q ranges, fixed-slice map task templates and cumulative partial counts, the way
    `Selector::select_partitioned` materialises them (attn/gqa/sdpa.rs:476-550,780-819)."""
    ranges, templates, cu = [], [], [0]
    flat = 0
    for history, n in zip(histories, q_lens):
        begin = flat
        while begin < flat + n:
            end = min(begin + max_q_tokens, flat + n)
            visible = history + (end - flat)
            index = len(ranges)
            ranges.append((begin, end))
            splits = max((visible + kv_slice - 1) // kv_slice, 0)
            for s in range(splits):
                templates.append((index, s * kv_slice, min((s + 1) * kv_slice, visible)))
            cu.append(len(templates))
            begin = end
        flat += n
    return (np.asarray(ranges, dtype=np.uint32).reshape(-1, 2), np.asarray(templates, dtype=np.uint32).reshape(-1, 3),
            np.asarray(cu, dtype=np.uint32))


def expected_output(w: Workload, threads: int = 8) -> np.ndarray:
    return oracle.paged_gqa(w.geom, w.q_bits, w.kv_pages, w.req_slots, w.page_ids, w.visible, layer=w.layer,
                            num_threads=threads)


# Parity gate: bf16 in, f32 accumulate, bf16 out.  |a - e| <= 2e-3 + 1e-2 * |e| per element.
ABS_TOL = 2.0e-3
REL_TOL = 1.0e-2


def assert_parity(actual: np.ndarray, expected: np.ndarray, what: str = "", abs_tol: float = ABS_TOL,
                  rel_tol: float = REL_TOL) -> dict:
    actual = np.asarray(actual, dtype=np.float32).reshape(-1)
    expected = np.asarray(expected, dtype=np.float32).reshape(-1)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    assert np.isfinite(actual).all(), f"{what}: non-finite values in the output"
    error = np.abs(actual - expected)
    bound = abs_tol + rel_tol * np.abs(expected)
    worst = int(np.argmax(error - bound))
    stats = {
        "max_abs": float(error.max(initial=0.0)),
        "mean_abs": float(error.mean()) if error.size else 0.0,
        "max_rel": float((error / np.maximum(np.abs(expected), 1e-6))[np.abs(expected) > 0.05].max(initial=0.0)),
    }
    assert (error <= bound).all(), (
        f"{what}: element {worst}: actual={actual[worst]} expected={expected[worst]} "
        f"|diff|={error[worst]} bound={bound[worst]} stats={stats}")
    return stats


# The north-star gate on the arithmetic itself: both bounds at once, on the f32 result before the bf16 output cast
# (a bf16 cast alone is off by up to 2^-9 |o|, which exceeds 2e-3 for |o| > 1).  The relative error is taken over
# elements with |expected| > 0.05, as the stats of `assert_parity` report it.
def assert_strict_parity(actual: np.ndarray, expected: np.ndarray, what: str = "") -> dict:
    actual = np.asarray(actual, dtype=np.float32).reshape(-1)
    expected = np.asarray(expected, dtype=np.float32).reshape(-1)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    assert np.isfinite(actual).all(), f"{what}: non-finite values in the output"
    error = np.abs(actual - expected)
    sizeable = np.abs(expected) > 0.05
    relative = error[sizeable] / np.abs(expected[sizeable])
    stats = {
        "max_abs": float(error.max(initial=0.0)),
        "mean_abs": float(error.mean()) if error.size else 0.0,
        "max_rel": float(relative.max(initial=0.0)),
        "elements": int(error.size),
    }
    assert stats["max_abs"] <= ABS_TOL, f"{what}: max abs error {stats['max_abs']} > {ABS_TOL} ({stats})"
    assert stats["max_rel"] <= REL_TOL, f"{what}: max relative error {stats['max_rel']} > {REL_TOL} ({stats})"
    return stats


def record_parity(name: str, stats: dict, path: str | None = None) -> None:
    """Appends one JSON line (case name + error statistics) to the parity log of this test run."""
    import json
    import os

    path = path or os.environ.get("KHM_PARITY_LOG") or os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                                                     "gpurun_out", "parity_stats.jsonl")
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "a") as handle:
            handle.write(json.dumps({"case": name, **stats}) + "\n")
    except OSError:
        pass   # a read-only tree keeps the printed statistics only
