"""One attention layer's worth of the path on one stream, with no host synchronisation in between, as GQA::record enqueues
it (crates/inference-executor-metal/src/attn/gqa/backend.rs:382-421,438-542): per-head RMSNorm + RoPE of the new tokens' Q
rows, RMSNorm + RoPE of their K rows fused with the K/V page write, then the SDPA over the cached history and the rows that
were just written (a chunked prefill onto a paged prefix, a speculative block and a single decoded token in one batch).
Every stage is checked against the oracle's chain of the same stages, and the attention also against the oracle run on
exactly the bytes the producers left in memory.  The page bytes travel from one launch to the next through streaming stores and streaming loads."""
import dataclasses

import numpy as np
import pytest
import torch

from khalamari_amd import k_norm_rope_page_write as fused_writer
from khalamari_amd import kv_page_write as kpw
from khalamari_amd import rms_norm_rope as rnr
from khalamari_amd import sdpa, sliced_q
from khalamari_amd._lib import DTYPE_BF16, DTYPE_FP8_E4M3FN, ReplayU32
from oracle import gqa_oracle as oracle

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu

EPS, THETA = 1e-6, 10_000_000.0


@pytest.mark.parametrize("fp8_pages", [True, False])
@pytest.mark.parametrize("hq,hkv,d,tile", [(16, 2, 128, 32), (12, 2, 256, 32), (16, 2, 128, 8)])
def test_norm_rope_page_write_then_attend_on_one_stream(device, fp8_pages, hq, hkv, d, tile):
    histories, q_lens = [300, 0, 1000, 77], [40, 17, 5, 1]
    tpp = 16
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories, q_lens=q_lens,
                              seed=900 + d + tile, fp8_pages=fp8_pages, garbage_bits=(0x7F if fp8_pages else 0x7FC0))
    g = w.geom
    rng = np.random.default_rng(901)
    total = w.num_tokens
    q_raw = oracle.f32_to_bf16_bits((rng.standard_normal((total, hq, d)) * 2).astype(np.float32))
    k_raw = oracle.f32_to_bf16_bits((rng.standard_normal((total, hkv, d)) * 2).astype(np.float32))
    v_new = oracle.f32_to_bf16_bits(rng.standard_normal((total, hkv, d)).astype(np.float32))
    weight_q = oracle.f32_to_bf16_bits((0.75 + rng.random(d) * 0.5).astype(np.float32))
    weight_k = oracle.f32_to_bf16_bits((0.75 + rng.random(d) * 0.5).astype(np.float32))
    positions = np.concatenate([h + np.arange(n) for h, n in zip(histories, q_lens)]).astype(np.uint32)

    # the oracle's chain: norm + rope of Q and K, K/V rows into the pages, attention over the pages
    q_expected = oracle.rms_norm_rope(q_raw, weight_q, positions, hq, d, d, EPS, THETA, io_bf16=True, weight_bf16=True)
    k_expected = oracle.rms_norm_rope(k_raw, weight_k, positions, hkv, d, d, EPS, THETA, io_bf16=True, weight_bf16=True)
    pages_expected = oracle.kv_page_write(w.kv_pages.reshape(-1), k_expected, v_new, w.req_slots, positions, w.page_ids, total, w.layer,
                                          g.num_gqa_layers, g.num_blocks, g.num_page_ids_per_block, hkv, d, tpp, g.page_bytes, fp8_pages)
    expected = helpers.expected_output(dataclasses.replace(w, q_bits=q_expected, kv_pages=pages_expected.reshape(w.kv_pages.shape)))

    # the device: the pool holds the histories; the rows of the new tokens hold what the workload generator put there and
    # are overwritten by the fused writer
    to = lambda a: gpu_runner.to_device(np.ascontiguousarray(a), device)  # noqa: E731
    pages = to(w.kv_pages)
    positions_d, slots_d, table_d = to(positions), to(w.req_slots), to(w.page_ids)
    q_rows = torch.zeros(total * hq * d, dtype=torch.int16, device=device)
    norm_q = rnr.Config.bf16(hq, d, d, EPS, THETA).with_norm_weight_dtype(DTYPE_BF16)
    norm_k = rnr.Config.bf16(hkv, d, d, EPS, THETA).with_norm_weight_dtype(DTYPE_BF16)
    kv_dtype = DTYPE_FP8_E4M3FN if fp8_pages else DTYPE_BF16
    page_config = kpw.Config(hkv, d, g.page_bytes, kv_dtype=kv_dtype)
    page_shape = kpw.Shape(total, kpw.PageTableLayout(w.num_req_slots, g.num_gqa_layers, g.num_blocks, g.num_page_ids_per_block))

    config = gpu_runner.component_config(w, sliced_q.Config)
    ratio = hq // hkv
    variant = sdpa.ExecutionVariant.sliced_q(config.sdpa_config(), sdpa.MAP_Q_TOKENS_AND_HEADS, tile, 64, ratio)
    ranges, templates, _ = helpers.fixed_slice_plan(histories, q_lens, tile, 1 << 30)
    ranges = np.asarray(ranges, dtype=np.uint32).reshape(-1, 2)
    templates = np.asarray(templates, dtype=np.uint32).reshape(-1, 3)
    shape = sliced_q.Shape(total, ranges.shape[0], templates.shape[0])
    compute = sliced_q.Compute(config, variant, shape, direct=True)
    out = torch.full((total, hq, d), 0x4228, dtype=torch.int16, device=device)
    visible_d, ranges_d, templates_d = to(w.visible), to(ranges), to(templates)
    weight_q_d, weight_k_d, q_raw_d, k_raw_d, v_new_d = to(weight_q), to(weight_k), to(q_raw), to(k_raw), to(v_new)
    torch.cuda.synchronize()

    print(f"append then attend: Hq{hq}/Hkv{hkv}/D{d} tile {tile} fp8_pages={fp8_pages}", flush=True)
    rnr.Compute(norm_q).invoke(rnr.Shape(total), input=q_raw_d, norm_weight=weight_q_d, flat_token_indices=positions_d, output=q_rows,
                               num_active_tokens=ReplayU32.fixed(total))
    fused_writer.Compute(norm_k, page_config).invoke(page_shape, pages=pages, k=k_raw_d, v=v_new_d, norm_weight=weight_k_d, req_slots=slots_d,
                                                     flat_token_indices=positions_d, page_ids=table_d, num_active_tokens=ReplayU32.fixed(total),
                                                     page_table_index=ReplayU32.fixed(w.layer))
    compute.invoke_direct(q=q_rows, kv_pages=pages, req_slots=slots_d, page_ids=table_d, visible_kv_token_ranges=visible_d,
                          q_token_ranges=ranges_d, sdpa_map_task_templates=templates_d, output=out, page_table_index=ReplayU32.fixed(w.layer),
                          num_active_tokens=ReplayU32.fixed(total), num_active_q_token_tiles=ReplayU32.fixed(ranges.shape[0]))
    torch.cuda.synchronize()

    # Producers against the oracle: the same rounding points, so nearly every bf16 value is the oracle's (an ulp of
    # 1/rms or of a sine can move a value across one rounding boundary: tests/test_rms_norm_rope.py bounds that); the V
    # bytes of the written rows are exact, and no byte outside the new tokens' rows has changed.
    q_device = q_rows.cpu().numpy().view(np.uint16).reshape(q_expected.shape)
    pages_device = pages.cpu().numpy().view(np.uint8).reshape(-1)
    assert np.mean(q_device == q_expected) > 0.99

    def written(k_bits, v_bits):   # the pool after writes of constant rows: 1.0 and -2.0 differ in every byte of both page formats
        rows = lambda bits: np.full((total, hkv, d), bits, dtype=np.uint16)  # noqa: E731
        return oracle.kv_page_write(np.zeros_like(pages_device), rows(k_bits), rows(v_bits), w.req_slots, positions, w.page_ids, total, w.layer,
                                    g.num_gqa_layers, g.num_blocks, g.num_page_ids_per_block, hkv, d, tpp, g.page_bytes, fp8_pages)
    one, minus_two = 0x3F80, 0xC000
    k_bytes = written(one, one) != written(minus_two, one)
    v_bytes = written(one, one) != written(one, minus_two)
    original, wanted = w.kv_pages.reshape(-1), pages_expected.reshape(-1)
    assert k_bytes.sum() == v_bytes.sum() == total * hkv * d * g.kv_element_bytes and not np.any(k_bytes & v_bytes)
    assert np.array_equal(pages_device[~(k_bytes | v_bytes)], original[~(k_bytes | v_bytes)])
    assert np.array_equal(pages_device[v_bytes], wanted[v_bytes])
    assert np.mean(pages_device[k_bytes] == wanted[k_bytes]) > 0.99

    # Attention against the oracle on exactly the bytes the device produced: the Q rows and the pages went from launch to
    # launch on the stream; the oracle reads what is in memory afterwards.
    expected_from_device = helpers.expected_output(dataclasses.replace(w, q_bits=q_device, kv_pages=pages_device.reshape(w.kv_pages.shape)))
    actual = gpu_runner.bf16_tensor_to_f32(out)
    helpers.assert_parity(actual, expected_from_device, "attention over the rows the producers just wrote")
    # and the whole chain against the oracle's chain, where a moved bf16 rounding in Q or K shows as a slightly different score
    helpers.assert_parity(actual, expected, "norm + rope, page write, attention on one stream", abs_tol=4e-3)


@pytest.mark.parametrize("one_launch_prologue", [False, True])
@pytest.mark.parametrize("fp8_pages", [True, False])
@pytest.mark.parametrize("hq,hkv,d,tile", [(16, 2, 128, 32), (12, 2, 256, 8)])
def test_layer_from_the_projection_rows_to_the_gated_output_on_one_stream(device, fp8_pages, hq, hkv, d, tile, one_launch_prologue):
    """Everything GQA::record enqueues between the input and the output projection (backend.rs:358-421) on one stream with
    no host synchronisation: the split of the gated projection rows into q, g, k, v, Q norm + RoPE, the fused K norm + RoPE
    + K/V page write (three launches, or khm_gqa_projection_norm_rope_page_write as one), and the SDPA with the sigmoid
    gate applied where the output is written: two launches for the layer in the shortest form."""
    from khalamari_amd import projection_norm_rope_page_write, qgkv_split

    histories, q_lens = [300, 0, 1000, 77], [40, 17, 5, 1]
    tpp = 16
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories, q_lens=q_lens,
                              seed=950 + d + tile, fp8_pages=fp8_pages, garbage_bits=(0x7F if fp8_pages else 0x7FC0))
    g = w.geom
    rng = np.random.default_rng(951)
    total = w.num_tokens
    bits = lambda shape, scale: oracle.f32_to_bf16_bits((rng.standard_normal(shape) * scale).astype(np.float32))  # noqa: E731
    q_raw, gate_bits = bits((total, hq, d), 2.0), bits((total, hq, d), 1.5)
    k_raw, v_new = bits((total, hkv, d), 2.0), bits((total, hkv, d), 1.0)
    # a projection row: [Hq x (q head | gate head)][Hkv x k head][Hkv x v head] (gqa_qgkv_split.metal:24-43)
    projection = np.concatenate([np.stack([q_raw, gate_bits], axis=2).reshape(total, 2 * hq * d), k_raw.reshape(total, -1),
                                 v_new.reshape(total, -1)], axis=1)
    weight_q = oracle.f32_to_bf16_bits((0.75 + rng.random(d) * 0.5).astype(np.float32))
    weight_k = oracle.f32_to_bf16_bits((0.75 + rng.random(d) * 0.5).astype(np.float32))
    positions = np.concatenate([h + np.arange(n) for h, n in zip(histories, q_lens)]).astype(np.uint32)

    to = lambda a: gpu_runner.to_device(np.ascontiguousarray(a), device)  # noqa: E731
    pages = to(w.kv_pages)
    positions_d, slots_d, table_d = to(positions), to(w.req_slots), to(w.page_ids)
    rows = lambda heads: torch.full((total, heads, d), 0x4228, dtype=torch.int16, device=device)  # noqa: E731
    q_split, g_split, k_split, v_split, q_rows, out = rows(hq), rows(hq), rows(hkv), rows(hkv), rows(hq), rows(hq)
    norm_q = rnr.Config.bf16(hq, d, d, EPS, THETA).with_norm_weight_dtype(DTYPE_BF16)
    norm_k = rnr.Config.bf16(hkv, d, d, EPS, THETA).with_norm_weight_dtype(DTYPE_BF16)
    page_config = kpw.Config(hkv, d, g.page_bytes, kv_dtype=DTYPE_FP8_E4M3FN if fp8_pages else DTYPE_BF16)
    page_shape = kpw.Shape(total, kpw.PageTableLayout(w.num_req_slots, g.num_gqa_layers, g.num_blocks, g.num_page_ids_per_block))
    config = gpu_runner.component_config(w, sliced_q.Config)
    variant = sdpa.ExecutionVariant.sliced_q(config.sdpa_config(), sdpa.MAP_Q_TOKENS_AND_HEADS, tile, 64, hq // hkv)
    ranges, templates, _ = helpers.fixed_slice_plan(histories, q_lens, tile, 1 << 30)
    ranges = np.asarray(ranges, dtype=np.uint32).reshape(-1, 2)
    templates = np.asarray(templates, dtype=np.uint32).reshape(-1, 3)
    compute = sliced_q.Compute(config, variant, sliced_q.Shape(total, ranges.shape[0], templates.shape[0]), direct=True)
    visible_d, ranges_d, templates_d = to(w.visible), to(ranges), to(templates)
    weight_q_d, weight_k_d, projection_d = to(weight_q), to(weight_k), to(projection)
    torch.cuda.synchronize()

    print(f"projection to gated output: Hq{hq}/Hkv{hkv}/D{d} tile {tile} fp8_pages={fp8_pages}", flush=True)
    active = ReplayU32.fixed(total)
    if one_launch_prologue:
        projection_norm_rope_page_write.Compute(norm_q, norm_k, page_config).invoke(
            page_shape, projection=projection_d, q_norm_weight=weight_q_d, k_norm_weight=weight_k_d, q_output=q_rows, gate_output=g_split,
            pages=pages, req_slots=slots_d, flat_token_indices=positions_d, page_ids=table_d, num_active_tokens=active,
            page_table_index=ReplayU32.fixed(w.layer))
    else:
        qgkv_split.Compute(qgkv_split.Config.bf16(hq, hkv, d)).invoke(qgkv_split.Shape(total), qgkv=projection_d, q=q_split, g=g_split, k=k_split,
                                                                        v=v_split, num_active_tokens=active)
        rnr.Compute(norm_q).invoke(rnr.Shape(total), input=q_split, norm_weight=weight_q_d, flat_token_indices=positions_d, output=q_rows,
                                   num_active_tokens=active)
        fused_writer.Compute(norm_k, page_config).invoke(page_shape, pages=pages, k=k_split, v=v_split, norm_weight=weight_k_d, req_slots=slots_d,
                                                         flat_token_indices=positions_d, page_ids=table_d, num_active_tokens=active,
                                                         page_table_index=ReplayU32.fixed(w.layer))
    compute.invoke_direct(q=q_rows, kv_pages=pages, req_slots=slots_d, page_ids=table_d, visible_kv_token_ranges=visible_d,
                          q_token_ranges=ranges_d, sdpa_map_task_templates=templates_d, output=out, page_table_index=ReplayU32.fixed(w.layer),
                          num_active_tokens=active, num_active_q_token_tiles=ReplayU32.fixed(ranges.shape[0]), gates=g_split)
    torch.cuda.synchronize()

    host = lambda t: t.cpu().numpy().view(np.uint16)  # noqa: E731
    assert np.array_equal(host(g_split), gate_bits)
    if not one_launch_prologue:
        assert np.array_equal(host(q_split), q_raw) and np.array_equal(host(k_split), k_raw) and np.array_equal(host(v_split), v_new)

    def gated(attention_f32):   # the gate sees the bf16-rounded attention output (gqa_activation_gate.metal:19-39)
        return oracle.bf16_bits_to_f32(oracle.gate_bf16(oracle.f32_to_bf16_bits(attention_f32).reshape(-1), gate_bits.reshape(-1)))

    actual = gpu_runner.bf16_tensor_to_f32(out)
    # the oracle on exactly the Q rows and page bytes the producers left in memory
    pages_device = pages.cpu().numpy().view(np.uint8).reshape(w.kv_pages.shape)
    from_device = helpers.expected_output(dataclasses.replace(w, q_bits=host(q_rows), kv_pages=pages_device))
    helpers.assert_parity(actual, gated(from_device), "gated attention over the rows the producers just wrote", abs_tol=4e-3)
    # and the oracle's own chain from the projection rows
    q_expected = oracle.rms_norm_rope(q_raw, weight_q, positions, hq, d, d, EPS, THETA, io_bf16=True, weight_bf16=True)
    k_expected = oracle.rms_norm_rope(k_raw, weight_k, positions, hkv, d, d, EPS, THETA, io_bf16=True, weight_bf16=True)
    pages_expected = oracle.kv_page_write(w.kv_pages.reshape(-1), k_expected, v_new, w.req_slots, positions, w.page_ids, total, w.layer,
                                          g.num_gqa_layers, g.num_blocks, g.num_page_ids_per_block, hkv, d, tpp, g.page_bytes, fp8_pages)
    chain = helpers.expected_output(dataclasses.replace(w, q_bits=q_expected, kv_pages=pages_expected.reshape(w.kv_pages.shape)))
    helpers.assert_parity(actual, gated(chain), "projection rows to gated output on one stream", abs_tol=6e-3)
