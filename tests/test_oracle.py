"""Pins the CPU oracle: reference known-answer tests, closed forms, an independent float64 brute force,
torch's scaled_dot_product_attention, and the invariants the domain fixes (page permutation, KV partition)."""
import math

import numpy as np
import pytest
import torch

from oracle import gqa_oracle as oracle

from . import helpers


def test_causal_attention_closed_form():
    # inference-executor-core/src/attn/gqa/reference.rs:84-115
    out = oracle.projected_gqa([0, 2], [0], [1, 0, 1, 0, 0, 2, 0, 2], [[1, 0, 0, 1]], [[10, 0, 0, 20]], 2, 1, 2, 1.0)
    f = np.float32
    first = f(np.exp(f(-2.0)))  # the reference builds its expectation in f32 as well
    total = f(first + f(1.0))
    w1, w2 = f(first / total), f(f(1.0) / total)
    expected = np.array([10, 0, 10, 0, f(10) * w1, f(20) * w2, f(10) * w1, f(20) * w2], dtype=np.float32)
    assert np.abs(out.reshape(-1) - expected).max() < 1e-6


def test_softmax_and_sigmoid_known_answers():
    # inference-executor-core/src/reference.rs:95-108
    out = oracle.softmax([0.0, math.log(3.0)])
    assert abs(out[0] - 0.25) < 1e-6 and abs(out[1] - 0.75) < 1e-6
    assert oracle.sigmoid(0.0) == 0.5
    with pytest.raises(ValueError):
        oracle.softmax([])


def test_fp8_fixed_encodings_and_saturation():
    # components/gqa/fp8.rs:68-88
    cases = [(0.0, 0x00), (-0.0, 0x80), (2.0 ** -9, 0x01), (2.0 ** -6, 0x08), (1.0, 0x38), (1.5, 0x3C), (448.0, 0x7E),
             (-448.0, 0xFE), (449.0, 0x7E), (-449.0, 0xFE), (float("inf"), 0x7E), (float("-inf"), 0xFE)]
    for value, expected in cases:
        bits = oracle.f32_to_bf16_bits(np.array([value], dtype=np.float32))
        assert int(oracle.bf16_bits_to_fp8(bits)[0]) == expected, value
    nan_bits = oracle.f32_to_bf16_bits(np.array([np.nan], dtype=np.float32))
    assert int(oracle.bf16_bits_to_fp8(nan_bits)[0]) & 0x7F == 0x7F


def test_fp8_ties_to_even_round_trip_and_error_bounds():
    # fp8.rs:90-139
    enc = lambda v: int(oracle.bf16_bits_to_fp8(oracle.f32_to_bf16_bits(np.array([v], dtype=np.float32)))[0])
    assert enc(1.0625) == enc(1.0)
    assert enc(1.1875) == enc(1.25)
    table = oracle.fp8_decode_table()
    for code in range(256):
        if code & 0x7F == 0x7F:
            continue
        assert int(oracle.bf16_bits_to_fp8(np.array([table[code]], dtype=np.uint16))[0]) == code
    min_normal = 2.0 ** -6
    sub = (np.arange(4097, dtype=np.float32) * np.float32(min_normal) / np.float32(4096.0)).astype(np.float32)
    src = oracle.bf16_round(sub)
    assert np.abs(oracle.fp8_round_trip(sub) - src).max() <= 2.0 ** -10
    normal = (np.float32(min_normal) + np.arange(458737, dtype=np.float32) / np.float32(1024.0)).astype(np.float32)
    normal = normal[normal <= 448.0]
    src = oracle.bf16_round(normal)
    assert (np.abs(oracle.fp8_round_trip(normal) - src) / src).max() <= 0.0625


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    values = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0,
                             np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], dtype=np.float32)])
    ours = oracle.f32_to_bf16_bits(values)
    theirs = torch.from_numpy(values).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, theirs)


def _float64_paged(w):
    g = w.geom
    pages = w.kv_pages.view(np.uint16).reshape(-1, 2, g.num_kv_heads, g.tokens_per_page, g.head_dim)
    table = w.page_ids.reshape(w.num_req_slots, g.num_gqa_layers, -1)
    q = oracle.bf16_bits_to_f32(w.q_bits).astype(np.float64)
    out = np.zeros((w.num_tokens, g.num_q_heads, g.head_dim), dtype=np.float64)
    ratio = g.num_q_heads // g.num_kv_heads
    for t in range(w.num_tokens):
        lo, hi = int(w.visible[t, 0]), int(w.visible[t, 1])
        if hi <= lo:
            continue
        tokens = np.arange(lo, hi)
        ids = table[w.req_slots[t], w.layer, tokens // g.tokens_per_page]
        k = oracle.bf16_bits_to_f32(pages[ids, 0, :, tokens % g.tokens_per_page, :]).astype(np.float64)
        v = oracle.bf16_bits_to_f32(pages[ids, 1, :, tokens % g.tokens_per_page, :]).astype(np.float64)
        for h in range(g.num_q_heads):
            s = k[:, h // ratio, :] @ q[t, h] * g.scale
            p = np.exp(s - s.max())
            out[t, h] = (p / p.sum()) @ v[:, h // ratio, :]
    return out


@pytest.mark.parametrize("tpp,ppb,layers", [(16, 1, 1), (8, 2, 2), (32, 1, 1), (4, 3, 1)])
def test_paged_oracle_matches_float64_brute_force(tpp, ppb, layers):
    w = helpers.make_workload(num_q_heads=6, num_kv_heads=2, head_dim=32, tokens_per_page=tpp, histories=[37, 0, 5],
                              q_lens=[2, 1, 4], seed=11, num_layers=layers, layer=layers - 1, page_ids_per_block=ppb)
    assert np.abs(helpers.expected_output(w, threads=2) - _float64_paged(w)).max() < 2e-6


def test_paged_oracle_matches_torch_sdpa():
    w = helpers.make_workload(num_q_heads=8, num_kv_heads=2, head_dim=64, tokens_per_page=16, histories=[200], q_lens=[7], seed=5)
    g = w.geom
    pages = w.kv_pages.view(np.uint16).reshape(-1, 2, g.num_kv_heads, 16, 64)
    ids = w.page_ids.reshape(-1)[: (207 + 15) // 16]
    k = oracle.bf16_bits_to_f32(pages[ids, 0]).transpose(1, 0, 2, 3).reshape(2, -1, 64)[:, :207]
    v = oracle.bf16_bits_to_f32(pages[ids, 1]).transpose(1, 0, 2, 3).reshape(2, -1, 64)[:, :207]
    q = torch.from_numpy(oracle.bf16_bits_to_f32(w.q_bits)).permute(1, 0, 2)  # [Hq, T, D]
    kk = torch.from_numpy(k.copy()).repeat_interleave(4, dim=0)
    vv = torch.from_numpy(v.copy()).repeat_interleave(4, dim=0)
    mask = torch.arange(207)[None, :] < torch.from_numpy(w.visible[:, 1].astype(np.int64))[:, None]
    ref = torch.nn.functional.scaled_dot_product_attention(q[None], kk[None], vv[None], attn_mask=mask[None, None], scale=g.scale)
    assert np.abs(helpers.expected_output(w) - ref[0].permute(1, 0, 2).numpy()).max() < 2e-6


def test_windowed_and_empty_visible_ranges():
    # sliced_q_test.rs:179-205: a window [begin, end) equals dense attention over that slice; empty -> zeros
    w = helpers.make_workload(num_q_heads=4, num_kv_heads=2, head_dim=16, tokens_per_page=8, histories=[30], q_lens=[3], seed=2)
    w.visible[0] = (28, 31)
    w.visible[1] = (7, 7)
    w.visible[2] = (0, 33)
    out = helpers.expected_output(w)
    assert np.abs(out - _float64_paged(w)).max() < 2e-6
    assert np.all(out[1] == 0.0)


def test_output_is_invariant_under_page_permutation():
    a = helpers.make_workload(num_q_heads=4, num_kv_heads=2, head_dim=32, tokens_per_page=16, histories=[100, 17], q_lens=[1, 2],
                              seed=3, permute=False)
    b = helpers.make_workload(num_q_heads=4, num_kv_heads=2, head_dim=32, tokens_per_page=16, histories=[100, 17], q_lens=[1, 2],
                              seed=3, permute=True)
    # same generator state up to the permutation draw is not guaranteed; compare against float64 instead of each other
    assert np.abs(helpers.expected_output(a) - _float64_paged(a)).max() < 2e-6
    assert np.abs(helpers.expected_output(b) - _float64_paged(b)).max() < 2e-6
    # and physically re-permuting the same pages with a consistent table leaves the result bit-identical
    perm = np.random.default_rng(9).permutation(b.kv_pages.shape[0])
    inverse = np.argsort(perm)
    moved = helpers.Workload(b.geom, b.q_bits, b.kv_pages[perm], np.where(b.page_ids == helpers.U32_MAX, helpers.U32_MAX,
                             inverse[np.minimum(b.page_ids, len(perm) - 1)]).astype(np.uint32), b.req_slots, b.visible,
                             b.cu_tokens, b.token_indices, b.num_req_slots)
    assert np.array_equal(helpers.expected_output(moved), helpers.expected_output(b))


@pytest.mark.parametrize("kv_slice", [1, 7, 16, 64, 1000])
def test_any_kv_partition_merges_to_the_unsplit_result(kv_slice):
    # attn/gqa/sdpa_test.rs:462-498 (coverage) + docs/gqa_sdpa_selection.md:449-458 (merge algebra)
    histories, q_lens = [45, 3], [3, 2]
    w = helpers.make_workload(num_q_heads=4, num_kv_heads=2, head_dim=16, tokens_per_page=8, histories=histories, q_lens=q_lens, seed=4)
    expected = helpers.expected_output(w)
    # sliced-Q flavour (ranges of up to 2 tokens)
    ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 2, kv_slice)
    sums, maxs, partial = oracle.map_partials(w.geom, templates, ranges, 2, w.q_bits, w.kv_pages, w.req_slots, w.page_ids, w.visible)
    merged = oracle.reduce_sliced_q(np.nan_to_num(sums), np.nan_to_num(maxs, neginf=-np.inf), np.nan_to_num(partial), ranges, cu, 2,
                                    w.num_tokens, 4, 16)
    assert np.abs(merged - expected).max() < 2e-6
    # sliced-KV flavour (one token per range)
    ranges1, templates1, cu1 = helpers.fixed_slice_plan(histories, q_lens, 1, kv_slice)
    sums, maxs, partial = oracle.map_partials(w.geom, templates1, ranges1, 1, w.q_bits, w.kv_pages, w.req_slots, w.page_ids, w.visible)
    merged = oracle.reduce_sliced_kv(sums[..., 0], maxs[..., 0], partial[:, :, 0], cu1, w.num_tokens, 4, 16)
    assert np.abs(merged - expected).max() < 2e-6


def test_empty_partial_is_canonical_and_ignored_by_reduce():
    # docs/executor_gqa.md:643-646, sliced_q_test.rs:511-514
    w = helpers.make_workload(num_q_heads=2, num_kv_heads=1, head_dim=8, tokens_per_page=8, histories=[0], q_lens=[3], seed=6)
    ranges = np.array([[0, 3]], dtype=np.uint32)
    templates = np.array([[0, 0, 0], [0, 0, 3], [0xFFFFFFFF] * 3], dtype=np.uint32)
    sums, maxs, partial = oracle.map_partials(w.geom, templates, ranges, 4, w.q_bits, w.kv_pages, w.req_slots, w.page_ids, w.visible)
    assert np.all(sums[0, :, :3] == 0) and np.all(np.isneginf(maxs[0, :, :3])) and np.all(partial[0, :, :3] == 0)
    assert np.isnan(sums[2]).all() and np.isnan(sums[:, :, 3]).all()  # sentinel template / inactive token untouched
    merged = oracle.reduce_sliced_q(np.nan_to_num(sums), np.nan_to_num(maxs, neginf=-np.inf), np.nan_to_num(partial), ranges, [0, 2], 4, 3, 2, 8)
    assert np.abs(merged - helpers.expected_output(w)).max() < 2e-6


def test_gate_known_answers():
    # activation_gate.rs:198-250: f32 gate = a / (1 + exp(-g)), tolerance 2e-5
    a = (np.arange(32, dtype=np.float32) * 0.03125 - 0.5).astype(np.float32)
    g = (np.arange(32, dtype=np.float32) * -0.0625 + 0.75).astype(np.float32)
    assert np.abs(oracle.gate_f32(a, g) - a / (1.0 + np.exp(-g.astype(np.float64)))).max() < 2e-5
    # bf16 build: independent numpy restatement of gqa_activation_gate.metal:19-26 over every bf16 gate value
    gate_bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = oracle.bf16_bits_to_f32(gate_bits)
    finite = np.isfinite(x)
    r = oracle.bf16_round
    with np.errstate(over="ignore"):
        y = r(1.0 / r(1.0 + r(np.exp(r(-r(np.abs(x)))).astype(np.float32))))
    sig = np.where(x < 0, r(1.0 - y), y)
    attn = oracle.f32_to_bf16_bits(np.full(65536, 1.5, dtype=np.float32))
    got = oracle.bf16_bits_to_f32(oracle.gate_bf16(attn, gate_bits))
    assert np.array_equal(got[finite], r(np.float32(1.5) * sig)[finite])
    assert abs(float(got[gate_bits == 0][0]) - 0.75) < 1e-6  # sigmoid(0) = .5


def _lcg_values(count, seed):
    """generated_values of the reference's fixtures (sliced_kv_test.rs:501-509): uniform in [-1, 1)."""
    out = np.empty(count, dtype=np.float32)
    state = seed
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(np.float32(state >> 8) / np.float32(16777216.0)) * np.float32(2.0) - np.float32(1.0)
    return out


def test_fp8_kv_output_quality_against_bf16_oracle():
    """test_fp8_kv_output_quality_against_bf16_oracle (sliced_kv_test.rs:68-115): a 64-token causal pass at the
    fixture geometry (Hq4/Hkv2/D2, scale 0.5) with K/V through the FP8 round trip stays within max 0.025 / mean 0.005
    of the same pass on the bf16 values."""
    hq, hkv, d, tokens = 4, 2, 2, 64
    q = oracle.bf16_round(_lcg_values(tokens * hq * d, 0x7E102041)).reshape(tokens, hq, d)
    k = oracle.bf16_round(_lcg_values(tokens * hkv * d, 0x7E102042)).reshape(tokens, hkv, d)
    v = oracle.bf16_round(_lcg_values(tokens * hkv * d, 0x7E102043)).reshape(tokens, hkv, d)
    assert np.abs(k).max() <= 448 and np.abs(v).max() <= 448
    outputs = []
    for fp8 in (False, True):
        geom = oracle.Geometry(hq, hkv, d, tokens, 0.5, 1, 1, 1, oracle.KV_FP8_E4M3FN if fp8 else oracle.KV_BF16)
        pages = oracle.pack_pages(geom, 1, [(k, v)], [[0]])
        visible = np.array([[0, i + 1] for i in range(tokens)], dtype=np.uint32)
        outputs.append(oracle.paged_gqa(geom, oracle.f32_to_bf16_bits(q), pages, np.zeros(tokens, dtype=np.uint32),
                                        np.zeros(1, dtype=np.uint32), visible))
    error = np.abs(outputs[1] - outputs[0])
    assert error.max() <= 0.025 and error.mean() <= 0.005, (error.max(), error.mean())
