"""GPU parity of the sliced-Q path (verify blocks, windowed ranges, direct output) and of replay parameters,
mirroring crates/inference-backend-metal/src/components/gqa/sdpa/sliced_q_test.rs and sliced_kv_test.rs."""
import numpy as np
import pytest
import torch

from khalamari_amd import activation_gate, batch_metadata, sdpa, sliced_kv, sliced_q
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, KhmError, ReplayU32
from khalamari_amd.selector import GQAReplayBucketPolicy, RequestShape, Selector
from oracle import gqa_oracle as oracle

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu

POISON = 0x4228  # bf16 42.0, as the reference poisons inactive outputs (sliced_q_test.rs:150,209-214)


def test_speculative_verify_blocks(device):
    """Config-4 shape at reduced context: q_len = 1 + k, k in 1..4, causal inside the block, Hq64/Hkv8/D128."""
    histories = [300, 4096, 77, 1029, 15]
    q_lens = [2, 5, 3, 4, 5]
    w = helpers.make_workload(num_q_heads=64, num_kv_heads=8, head_dim=128, tokens_per_page=16, histories=histories,
                              q_lens=q_lens, seed=21)
    expected = helpers.expected_output(w)
    for kv_slice, direct in [(512, False), (1 << 20, True), (100, False)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 8, kv_slice)
        print(f"verify kv_slice={kv_slice} direct={direct}", flush=True)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=8,
                                         max_q_heads=8, stage=64, direct=direct)
        helpers.assert_parity(actual, expected, f"verify slice={kv_slice} direct={direct}")


@pytest.mark.parametrize("head_dim,tpp", [(128, 8), (128, 16), (256, 8), (256, 16), (256, 32)])
def test_replay_paged_ranges(device, head_dim, tpp):
    """sliced_q_test.rs:57-217: two layers, two page ids per block, requests in swapped slots, windowed and empty
    visible ranges, inactive tokens keep their poison."""
    hq, hkv = 6, 2
    rng = np.random.default_rng(17)
    geom = oracle.Geometry(hq, hkv, head_dim, tpp, head_dim ** -0.5, num_gqa_layers=2, num_blocks=3, num_page_ids_per_block=2)
    contexts = [36, 7]
    keys = [oracle.bf16_round(rng.standard_normal((n, hkv, head_dim), dtype=np.float32) * 0.5) for n in contexts]
    values = [oracle.bf16_round(rng.standard_normal((n, hkv, head_dim), dtype=np.float32) * 0.5) for n in contexts]
    page_table = np.full((2, 2, 6), 0xFFFFFFFF, dtype=np.uint32)
    page_lists, next_page = [], 11
    for req, slot in enumerate([1, 0]):
        pages = []
        for p in range(-(-contexts[req] // tpp)):
            page_table[slot, 1, p] = next_page
            pages.append(next_page)
            next_page -= 1
        page_lists.append(pages)
    kv_pages = oracle.pack_pages(geom, 12, list(zip(keys, values)), page_lists, fill_bits=0x7FC0)
    q_bits = oracle.f32_to_bf16_bits(rng.standard_normal((20, hq, head_dim), dtype=np.float32) * 0.5)
    slots = np.ones(20, dtype=np.uint32)
    slots[17] = 0
    ranges = np.array([[0, 16], [16, 17], [17, 18], [0xFFFFFFFF, 0xFFFFFFFF]], dtype=np.uint32)
    templates = np.array([[0, 0, 16], [0, 16, 35], [1, 0, 16], [1, 16, 36], [2, 0, 7], [2, 7, 7],
                          [0xFFFFFFFF] * 3, [0xFFFFFFFF] * 3], dtype=np.uint32)
    cu = np.array([0, 2, 4, 6, 0xFFFFFFFF], dtype=np.uint32)
    layout = sliced_kv.Layout(2, 2, 3, 2)
    config = sliced_q.Config(hq, hkv, head_dim, geom.scale, geom.page_bytes, layout)
    shape = sliced_q.Shape(20, 4, 8)
    variant = sdpa.ExecutionVariant.sliced_q_per_head(config.sdpa_config(), 16, 16, 2)
    compute = sliced_q.Compute.new(config, variant, shape)
    dev = lambda a: gpu_runner.to_device(a, device)
    q, pages, slot_d, table, rng_d, tmpl, cu_d = map(dev, (q_bits, kv_pages, slots, page_table.reshape(-1), ranges, templates, cu))
    partial = torch.zeros(config.partial_output_bytes(variant, shape), dtype=torch.uint8, device=device)
    sums = torch.zeros(config.partial_output_stats_bytes(variant, shape), dtype=torch.uint8, device=device)
    maxs = torch.zeros_like(sums)
    for windowed in (False, True):
        visible = np.zeros((20, 2), dtype=np.uint32)
        for token in range(18):
            req = int(token == 17)
            end = 20 + token if req == 0 else 7
            begin = (end - 3 if req == 0 else end) if windowed else 0
            visible[token] = (begin, end)
        vis = dev(visible)
        out = torch.full((20, hq, head_dim), POISON, dtype=torch.int16, device=device)
        print(f"paged ranges d={head_dim} tpp={tpp} windowed={windowed}", flush=True)
        compute.invoke_map(q=q, kv_pages=pages, req_slots=slot_d, page_ids=table, visible_kv_token_ranges=vis, q_token_ranges=rng_d,
                           sdpa_map_task_templates=tmpl, partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                           page_table_index=ReplayU32.fixed(1), num_active_tokens=ReplayU32.fixed(18),
                           num_active_q_token_tiles=ReplayU32.fixed(3), num_active_kv_splits=ReplayU32.fixed(6))
        compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=rng_d,
                              cu_sdpa_partial_outputs=cu_d, output=out, num_active_q_token_tiles=ReplayU32.fixed(3))
        torch.cuda.synchronize()
        expected = oracle.paged_gqa(geom, q_bits[:18], kv_pages, slots[:18], page_table.reshape(-1), visible[:18], layer=1)
        actual = gpu_runner.bf16_tensor_to_f32(out)
        helpers.assert_parity(actual[:18], expected, f"paged ranges windowed={windowed}")
        if windowed:
            assert np.all(actual[17] == 0.0)  # empty visible range -> zeros
        assert np.all(out[18:].cpu().numpy() == POISON)  # inactive tokens untouched


@pytest.mark.parametrize("kind,ratio,tile,heads,stage,head_dim", [
    (sdpa.MAP_Q_HEADS_PER_TOKEN, 6, 4, 6, 8, 128),
    (sdpa.MAP_Q_TOKENS_AND_HEADS, 6, 4, 6, 16, 128),
    (sdpa.MAP_Q_TOKENS_AND_HEADS, 6, 4, 3, 32, 256),
    (sdpa.MAP_Q_HEADS_PER_TOKEN, 8, 2, 4, 64, 256),
    (sdpa.MAP_Q_TOKENS_AND_HEADS, 12, 4, 12, 128, 256),
    (sdpa.MAP_Q_TOKENS_PER_HEAD, 12, 1, 6, 64, 128),
    (sdpa.MAP_Q_TOKENS_PER_HEAD, 6, 32, 1, 8, 128),
    (sdpa.MAP_Q_HEADS_PER_TOKEN, 5, 4, 3, 64, 256),
    (sdpa.MAP_Q_HEADS_PER_TOKEN, 8, 32, 8, 128, 256),
    (sdpa.MAP_Q_TOKENS_AND_HEADS, 12, 16, 12, 64, 256),
    (sdpa.MAP_Q_TOKENS_AND_HEADS, 8, 16, 8, 64, 128),
    (sdpa.MAP_Q_TOKENS_AND_HEADS, 8, 32, 8, 64, 128),
])
def test_q_token_head_assignments_and_direct_output(device, kind, ratio, tile, heads, stage, head_dim):
    """sliced_q_test.rs:219-401: tile/head geometries x {split, direct}, reversed pages, windowed and empty ranges."""
    contexts = [280, 257] if stage >= 64 else [24, 9]
    hq, hkv, tpp = ratio * 2, 2, 8
    rng = np.random.default_rng(31)
    blocks = -(-contexts[0] // tpp)
    num_pages = 2 * blocks
    geom = oracle.Geometry(hq, hkv, head_dim, tpp, head_dim ** -0.5, 1, blocks, 1)
    keys = [oracle.bf16_round(rng.standard_normal((n, hkv, head_dim), dtype=np.float32) * 0.5) for n in contexts]
    values = [oracle.bf16_round(rng.standard_normal((n, hkv, head_dim), dtype=np.float32) * 0.5) for n in contexts]
    page_lists = [[num_pages - 1 - (req * blocks + p) for p in range(-(-contexts[req] // tpp))] for req in range(2)]
    kv_pages = oracle.pack_pages(geom, num_pages, list(zip(keys, values)), page_lists)
    page_table = np.arange(num_pages, dtype=np.uint32)[::-1].copy()
    q_bits = oracle.f32_to_bf16_bits(rng.standard_normal((7, hq, head_dim), dtype=np.float32) * 0.5)
    slots = np.array([0, 0, 0, 0, 0, 1, 1], dtype=np.uint32)
    visible = np.zeros((7, 2), dtype=np.uint32)
    for token in range(7):
        req = int(token >= 5)
        end = contexts[0] - 4 + token if req == 0 else contexts[1] - 1 + token - 5
        begin = end if token == 6 else (0 if token == 0 else end - 7)
        visible[token] = (begin, end)
    expected = oracle.paged_gqa(geom, q_bits, kv_pages, slots, page_table, visible)
    q_ranges = []
    for begin, end in [(0, 5), (5, 7)]:
        for first in range(begin, end, tile):
            q_ranges.append((first, min(first + tile, end)))
    w = helpers.Workload(geom, q_bits, kv_pages, page_table, slots, visible, np.array([0, 5, 7], dtype=np.uint32),
                         np.zeros(2, dtype=np.uint32), 2)
    for direct in (False, True):
        templates, cu = [], [0]
        for index, (first, last) in enumerate(q_ranges):
            end = contexts[0] - 5 + last if first < 5 else contexts[1] - 6 + last
            templates += [(index, 0, end)] if direct else [(index, 0, 8), (index, 8, end)]
            cu.append(len(templates))
        print(f"assignments kind={kind} ratio={ratio} tile={tile} heads={heads} stage={stage} d={head_dim} direct={direct}", flush=True)
        try:
            actual = gpu_runner.run_sliced_q(w, q_ranges, templates, cu, device, kind=kind, max_q_tokens=tile, max_q_heads=heads,
                                             stage=stage, direct=direct, poison=POISON)
        except KhmError as error:
            if error.status == -2:
                pytest.skip(f"no gfx950 kernel yet: {error.message}")
            raise
        helpers.assert_parity(actual, expected, f"kind={kind} tile={tile} heads={heads} direct={direct}")


def test_replay_parameters_across_active_counts(device):
    """sliced_kv_test.rs:117-184 and sliced_q_test.rs:433-521: one recorded launch pair, active counts from a device
    parameter block; outputs past the active count stay untouched; the empty first template is canonical."""
    hq, hkv, d, tpp = 8, 2, 128, 16
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=[0], q_lens=[8], seed=40)
    layout = sliced_kv.Layout(1, 1, w.geom.num_blocks, 1)
    dev = lambda a: gpu_runner.to_device(a, device)
    q, pages, slots, table = map(dev, (w.q_bits, w.kv_pages, w.req_slots, w.page_ids))
    params = torch.zeros(4, dtype=torch.int32, device=device)
    # sliced-KV: token i attends to [0, i+1)
    config = sliced_kv.Config(hq, hkv, d, w.geom.scale, w.geom.page_bytes, layout)
    shape = sliced_kv.Shape(8, 8)
    compute = sliced_kv.Compute(config, sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), 128, 128, 4), shape)
    scratch = sliced_kv.Scratch(device, config, shape)
    tmpl = dev(np.array([[i, 0, i + 1] for i in range(8)], dtype=np.uint32))
    cu = dev(np.arange(9, dtype=np.uint32))
    expected = helpers.expected_output(w)
    for active in [1, 8, 3, 7, 2, 6, 4, 5]:
        out = torch.full((8, hq, d), POISON, dtype=torch.int16, device=device)
        params.copy_(torch.tensor([active, active, 0, 0], dtype=torch.int32))
        print(f"sliced-KV replay active={active}", flush=True)
        compute.invoke_map(q=q, kv_pages=pages, req_slots=slots, page_ids=table, sdpa_map_task_templates=tmpl,
                           partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                           partial_output=scratch.partial_output, page_table_index=ReplayU32.fixed(0),
                           num_active_tokens=ReplayU32.parameter(0), num_active_kv_splits=ReplayU32.parameter(1),
                           replay_parameters=params)
        compute.invoke_reduce(partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                              partial_output=scratch.partial_output, cu_sdpa_partial_outputs=cu, output=out,
                              num_active_tokens=ReplayU32.parameter(0), replay_parameters=params)
        torch.cuda.synchronize()
        actual = gpu_runner.bf16_tensor_to_f32(out)
        helpers.assert_parity(actual[:active], expected[:active], f"sliced-KV active={active}")
        assert np.all(out[active:].cpu().numpy() == POISON)
    # sliced-Q: one range of `active` tokens, first template empty
    qconfig = sliced_q.Config(hq, hkv, d, w.geom.scale, w.geom.page_bytes, layout)
    qshape = sliced_q.Shape(8, 1, 2)
    variant = sdpa.ExecutionVariant.sliced_q_per_head(qconfig.sdpa_config(), 8, 16, 4)
    qcompute = sliced_q.Compute.new(qconfig, variant, qshape)
    partial = torch.zeros(qconfig.partial_output_bytes(variant, qshape), dtype=torch.uint8, device=device)
    sums = torch.zeros(qconfig.partial_output_stats_bytes(variant, qshape), dtype=torch.uint8, device=device)
    maxs = torch.zeros_like(sums)
    vis = dev(w.visible)
    cu2 = dev(np.array([0, 2], dtype=np.uint32))
    for active in [1, 4, 3, 2, 8]:
        rng_d = dev(np.array([[0, active]], dtype=np.uint32))
        tmpl2 = dev(np.array([[0, 0, 0], [0, 0, active]], dtype=np.uint32))
        out = torch.full((8, hq, d), POISON, dtype=torch.int16, device=device)
        params.copy_(torch.tensor([active, 1, 2, 0], dtype=torch.int32))
        print(f"sliced-Q replay active={active}", flush=True)
        qcompute.invoke_map(q=q, kv_pages=pages, req_slots=slots, page_ids=table, visible_kv_token_ranges=vis, q_token_ranges=rng_d,
                            sdpa_map_task_templates=tmpl2, partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                            page_table_index=ReplayU32.fixed(0), num_active_tokens=ReplayU32.parameter(0),
                            num_active_q_token_tiles=ReplayU32.parameter(1), num_active_kv_splits=ReplayU32.parameter(2),
                            replay_parameters=params)
        qcompute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=rng_d,
                               cu_sdpa_partial_outputs=cu2, output=out, num_active_q_token_tiles=ReplayU32.parameter(1),
                               replay_parameters=params)
        torch.cuda.synchronize()
        actual = gpu_runner.bf16_tensor_to_f32(out)
        helpers.assert_parity(actual[:active], expected[:active], f"sliced-Q active={active}")
        assert np.all(out[active:].cpu().numpy() == POISON)
        sums_host = sums.view(torch.float32).cpu().numpy().reshape(2, hq, 8)
        maxs_host = maxs.view(torch.float32).cpu().numpy().reshape(2, hq, 8)
        assert np.all(sums_host[0, :, :active] == 0.0) and np.all(np.isneginf(maxs_host[0, :, :active]))


def test_pipelines_reused_across_replay_capacities(device):
    """sliced_kv_test.rs:20-42, sliced_q_test.rs:21-48: kernel identity does not depend on the shape."""
    config = sliced_kv.Config(8, 2, 128, 0.1, 2 * 2 * 16 * 128 * 2)
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), 128, 128, 4)
    first = sliced_kv.Compute(config, variant, sliced_kv.Shape(8, 8))
    for tokens, templates in [(4, 4), (8, 16), (16, 16)]:
        other = sliced_kv.Compute(config, variant, sliced_kv.Shape(tokens, templates))
        assert other.map_kernel_id() == first.map_kernel_id() and other.reduce_kernel_id() == first.reduce_kernel_id()
    with pytest.raises(KhmError, match="GQA SDPA query/output exceeds the shader u32 count domain"):
        sliced_kv.Compute(config, variant, sliced_kv.Shape(1 << 30, 1))
    with pytest.raises(KhmError, match="GQA SplitKV SlicedQ supports only"):
        bad = sliced_q.Config(5, 1, 192, 0.1, 2 * 8 * 192 * 2)
        sliced_q.Compute.new(bad, sdpa.ExecutionVariant.sliced_q_per_head(sdpa.Config(DTYPE_BF16, 5, 1, 128, 8), 8, 16, 5),
                             sliced_q.Shape(8, 1, 1))


def test_fused_gate_and_standalone_gate(device):
    """Config-3 epilogue: output * sigmoid(gate), fused into the Reduce and as the separate elementwise kernel
    (activation_gate.rs:198-250; bf16 step rounding of gqa_activation_gate.metal:19-39)."""
    histories = [3000, 100]
    w = helpers.make_workload(num_q_heads=24, num_kv_heads=4, head_dim=256, tokens_per_page=16, histories=histories, q_lens=[1, 1], seed=50)
    _, templates, cu = helpers.fixed_slice_plan(histories, [1, 1], 1, 2048)
    rng = np.random.default_rng(51)
    gate_bits = oracle.f32_to_bf16_bits(rng.standard_normal((2, 24, 256), dtype=np.float32))
    plain, _ = gpu_runner.run_sliced_kv(w, templates, cu, device)
    fused, _ = gpu_runner.run_sliced_kv(w, templates, cu, device, gates=gate_bits)
    want = oracle.bf16_bits_to_f32(oracle.gate_bf16(oracle.f32_to_bf16_bits(plain), gate_bits))
    assert np.array_equal(fused, want.reshape(fused.shape))  # same bf16 attention value in, bit-exact gate out
    expected = oracle.gate_f32(helpers.expected_output(w), oracle.bf16_bits_to_f32(gate_bits))
    helpers.assert_parity(fused, expected, "gated decode", abs_tol=4e-3)
    # standalone kernel, bf16 and f32 builds
    attn = gpu_runner.to_device(oracle.f32_to_bf16_bits(plain), device)
    gates = gpu_runner.to_device(gate_bits, device)
    out = torch.zeros_like(attn)
    activation_gate.invoke(DTYPE_BF16, 24, 256, 2, attn, gates, out, ReplayU32.fixed(2))
    torch.cuda.synchronize()
    assert np.array_equal(gpu_runner.bf16_tensor_to_f32(out), want.reshape(plain.shape))
    a32 = (np.arange(8 * 4, dtype=np.float32) * 0.03125 - 0.5).reshape(8, 2, 2)
    g32 = (np.arange(8 * 4, dtype=np.float32) * -0.0625 + 0.75).reshape(8, 2, 2)
    for active in [1, 8, 3, 7, 2, 6, 4, 5]:
        out32 = torch.full((8, 2, 2), 7.0, dtype=torch.float32, device=device)
        activation_gate.invoke(DTYPE_F32, 2, 2, 8, torch.from_numpy(a32).to(device), torch.from_numpy(g32).to(device), out32,
                               ReplayU32.fixed(active))
        torch.cuda.synchronize()
        got = out32.cpu().numpy()
        assert np.abs(got[:active] - a32[:active] / (1.0 + np.exp(-g32[:active]))).max() < 2e-5
        assert np.all(got[active:] == 7.0)


@pytest.mark.parametrize("hq,hkv,d,tile,heads", [(24, 4, 256, 32, 6), (24, 4, 256, 8, 6), (64, 8, 128, 32, 8), (8, 2, 128, 4, 4), (6, 2, 128, 4, 3)])
def test_gate_fused_into_the_sliced_q_outputs(device, hq, hkv, d, tile, heads):
    """The gated layer in prefill and verify: the sigmoid gate applied where the sliced-Q path writes its output - the
    direct Map's epilogue, the ranged Reduce - must give, bit for bit, what the standalone gate kernel gives on the
    ungated bf16 output (GQA::record runs the gate right after the SDPA: backend.rs:413-421,
    gqa_activation_gate.metal:19-39).  Twelve- and eight-wave prefill tiles, verify tiles and the one-tile kernel."""
    histories = [700, 33, 1500]
    q_lens = [70, 5, 40] if tile >= 32 else [5, 2, 4]
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories, q_lens=q_lens,
                              seed=77 + tile)
    rng = np.random.default_rng(78)
    gate_bits = oracle.f32_to_bf16_bits((rng.standard_normal((w.num_tokens, hq, d)) * 2).astype(np.float32))
    for kv_slice, direct in [(1 << 20, True), (256, False)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, tile, kv_slice)
        run = lambda gates: gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS,  # noqa: E731
                                                    max_q_tokens=tile, max_q_heads=heads, stage=64, direct=direct, gates=gates)
        print(f"gated sliced-Q hq={hq} d={d} tile={tile}x{heads} direct={direct}", flush=True)
        plain, fused = run(None), run(gate_bits)
        want = oracle.bf16_bits_to_f32(oracle.gate_bf16(oracle.f32_to_bf16_bits(plain), gate_bits))
        assert np.array_equal(fused, want.reshape(fused.shape))
        attn = gpu_runner.to_device(oracle.f32_to_bf16_bits(plain), device)
        out = torch.zeros_like(attn)
        activation_gate.invoke(DTYPE_BF16, hq, d, w.num_tokens, attn, gpu_runner.to_device(gate_bits, device), out, ReplayU32.fixed(w.num_tokens))
        torch.cuda.synchronize()
        assert np.array_equal(gpu_runner.bf16_tensor_to_f32(out).reshape(fused.shape), fused)
    expected = oracle.gate_f32(helpers.expected_output(w), oracle.bf16_bits_to_f32(gate_bits))
    helpers.assert_parity(fused, expected, "gated sliced-Q against the gated oracle", abs_tol=4e-3)


def test_device_gate_matches_the_oracle_on_every_bf16_gate_value(device):
    """All 65 536 bf16 gate bit patterns, each against several attention values, bit for bit: the device evaluates the
    exponential with v_exp_f32, the oracle with libm, and every intermediate is rounded to bf16
    (gqa_activation_gate.metal:19-39), so the two can only differ where the two exponentials straddle a bf16 rounding
    boundary - and nowhere do they.  NaN gates must give NaN (payloads are not compared)."""
    gate_bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    rng = np.random.default_rng(52)
    attention_values = [np.full(65536, 0x3F80, dtype=np.uint16),                                   # 1.0: the sigmoid itself
                        np.full(65536, 0xC2F7, dtype=np.uint16),                                   # -123.5
                        oracle.f32_to_bf16_bits(rng.standard_normal(65536, dtype=np.float32)),
                        oracle.f32_to_bf16_bits(rng.standard_normal(65536, dtype=np.float32) * 1e-3)]
    gates = gpu_runner.to_device(gate_bits, device)
    for attention_bits in attention_values:
        attn = gpu_runner.to_device(attention_bits, device)
        out = torch.zeros_like(attn)
        activation_gate.invoke(DTYPE_BF16, 1, 256, 256, attn, gates, out, ReplayU32.fixed(256))
        torch.cuda.synchronize()
        got = out.cpu().numpy().view(np.uint16)
        want = oracle.gate_bf16(attention_bits, gate_bits)
        got_nan = (got & 0x7FFF) > 0x7F80
        want_nan = (want & 0x7FFF) > 0x7F80
        assert np.array_equal(got_nan, want_nan)
        different = np.flatnonzero((got != want) & ~want_nan)
        assert different.size == 0, (f"{different.size} gate patterns differ, first: gate=0x{gate_bits[different[0]]:04x} "
                                     f"attention=0x{attention_bits[different[0]]:04x} got=0x{got[different[0]]:04x} want=0x{want[different[0]]:04x}")


def test_selector_and_metadata_drive_the_kernels_end_to_end(device):
    """prepare (Selector::select -> GQAMetadataBuffers::update) then record (Map/Reduce or direct), as
    GQA::prepare / record_sdpa do (attn/gqa/backend.rs:255-286,438-542)."""
    hq, hkv, d, tpp = 32, 4, 128, 16
    cases = [([700, 90, 2047, 5], [1, 1, 1, 1]), ([1500, 64], [4, 2]), ([0, 300], [40, 3])]
    for histories, q_lens in cases:
        w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories,
                                  q_lens=q_lens, seed=60 + len(histories), req_slot_order=list(range(len(histories)))[::-1])
        layout = sliced_kv.Layout(w.num_req_slots, 1, w.geom.num_blocks, 1)
        sconfig = sdpa.Config(DTYPE_BF16, hq, hkv, d, tpp)
        selector = Selector.for_lookup(sconfig, 64, layout)
        limits = selector.limits()
        policy = GQAReplayBucketPolicy(64, limits.max_map_task_templates)
        shapes = RequestShape.from_batch(histories, list(w.cu_tokens))
        selection = selector.select(shapes, policy, 64)
        metadata = batch_metadata.GQAMetadataBuffers(64, limits.max_map_task_templates)
        slots_by_request = [int(w.req_slots[w.cu_tokens[r]]) for r in range(len(histories))]
        shape = metadata.update(slots_by_request, histories, list(w.cu_tokens), selection)
        variant = selection.variant()
        dev = lambda a: gpu_runner.to_device(a, device)
        q = torch.zeros((64, hq, d), dtype=torch.int16, device=device)
        q[:w.num_tokens] = dev(w.q_bits)
        pages, table = dev(w.kv_pages), dev(w.page_ids)
        out = torch.full((64, hq, d), POISON, dtype=torch.int16, device=device)
        print(f"end-to-end histories={histories} q_lens={q_lens} kind={variant.map_kind} direct={selection.direct_output()} "
              f"templates={shape.num_sdpa_map_task_templates}/{shape.num_total_sdpa_map_task_templates}", flush=True)
        if variant.map_kind == sdpa.MAP_SLICED_KV:
            config = sliced_kv.Config(hq, hkv, d, w.geom.scale, w.geom.page_bytes, layout)
            kshape = sliced_kv.Shape(shape.num_total_tokens, shape.num_total_sdpa_map_task_templates)
            compute = sliced_kv.Compute(config, variant, kshape)
            scratch = sliced_kv.Scratch(device, config, kshape)
            compute.invoke_map(q=q, kv_pages=pages, req_slots=metadata.req_slots(), page_ids=table,
                               sdpa_map_task_templates=metadata.sdpa_map_task_templates(), partial_exp_sums=scratch.partial_exp_sums,
                               partial_max_logits=scratch.partial_max_logits, partial_output=scratch.partial_output,
                               page_table_index=ReplayU32.fixed(0), num_active_tokens=ReplayU32.fixed(shape.num_tokens),
                               num_active_kv_splits=ReplayU32.fixed(shape.num_sdpa_map_task_templates))
            compute.invoke_reduce(partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                                  partial_output=scratch.partial_output, cu_sdpa_partial_outputs=metadata.cu_sdpa_partial_outputs(),
                                  output=out, num_active_tokens=ReplayU32.fixed(shape.num_tokens))
        else:
            config = sliced_q.Config(hq, hkv, d, w.geom.scale, w.geom.page_bytes, layout)
            qshape = sliced_q.Shape(shape.num_total_tokens, shape.num_total_q_token_tiles, shape.num_total_sdpa_map_task_templates)
            common = dict(q=q, kv_pages=pages, req_slots=metadata.req_slots(), page_ids=table,
                          visible_kv_token_ranges=metadata.visible_kv_token_ranges(), q_token_ranges=metadata.q_token_ranges(),
                          sdpa_map_task_templates=metadata.sdpa_map_task_templates(), page_table_index=ReplayU32.fixed(0),
                          num_active_tokens=ReplayU32.fixed(shape.num_tokens),
                          num_active_q_token_tiles=ReplayU32.fixed(shape.num_q_token_tiles))
            if selection.direct_output():
                sliced_q.Compute.new_direct(config, variant, qshape).invoke_direct(output=out, **common)
            else:
                compute = sliced_q.Compute.new(config, variant, qshape)
                partial = torch.zeros(config.partial_output_bytes(variant, qshape), dtype=torch.uint8, device=device)
                sums = torch.zeros(config.partial_output_stats_bytes(variant, qshape), dtype=torch.uint8, device=device)
                maxs = torch.zeros_like(sums)
                compute.invoke_map(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                                   num_active_kv_splits=ReplayU32.fixed(shape.num_sdpa_map_task_templates), **common)
                compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                                      q_token_ranges=metadata.q_token_ranges(), cu_sdpa_partial_outputs=metadata.cu_sdpa_partial_outputs(),
                                      output=out, num_active_q_token_tiles=ReplayU32.fixed(shape.num_q_token_tiles))
        torch.cuda.synchronize()
        actual = gpu_runner.bf16_tensor_to_f32(out)
        helpers.assert_parity(actual[:w.num_tokens], helpers.expected_output(w), f"end-to-end {histories} {q_lens}")
        assert np.all(out[w.num_tokens:].cpu().numpy() == POISON)


@pytest.mark.parametrize("hq,hkv,d,tile", [(64, 8, 128, 32), (32, 4, 128, 16), (24, 4, 256, 16), (16, 2, 256, 32), (24, 4, 256, 32),
                                           (12, 2, 256, 32)])
def test_chunked_prefill_onto_a_paged_prefix(device, hq, hkv, d, tile):
    """Config-5 shape at reduced size: causal chunks appended to paged prefixes (including an empty prefix), wide
    Q tiles on the LDS-shared K/V kernel, direct output and split-KV + Reduce."""
    histories = [0, 333, 1000]
    q_lens = [150, 64, 37]
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories,
                              q_lens=q_lens, seed=90 + tile, garbage_bits=0x7FC0)
    expected = helpers.expected_output(w)
    ratio = hq // hkv
    for kv_slice, direct in [(1 << 20, True), (256, False), (100, False)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, tile, kv_slice)
        print(f"prefill hq={hq} hkv={hkv} d={d} tile={tile} kv_slice={kv_slice} direct={direct}", flush=True)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=tile,
                                         max_q_heads=ratio, stage=64, direct=direct)
        helpers.assert_parity(actual, expected, f"prefill tile={tile} slice={kv_slice} direct={direct}")


@pytest.mark.parametrize("hq,hkv,d,tile", [(16, 2, 128, 32), (8, 2, 128, 32), (12, 2, 256, 32), (12, 2, 256, 16)])
def test_long_interior_runs_of_a_prefill_tile_checked_on_every_row(device, hq, hkv, d, tile):
    """Prefixes of several thousand keys, so that nearly all tiles of a block are interior ones that run in the
    steady-state loop of the direct-output builds (unconditional requests, weights that do not follow the largest
    score); every Q row is compared with the oracle, at prefixes that start the KV walk on and off a tile boundary."""
    histories = [5000, 1531, 4096]
    q_lens = [96, 70, 33]
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories,
                              q_lens=q_lens, seed=411, garbage_bits=0x7FC0)
    expected = helpers.expected_output(w)
    ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, tile, 1 << 20)
    print(f"long interior runs hq={hq} hkv={hkv} d={d} tile={tile}", flush=True)
    actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=tile,
                                     max_q_heads=hq // hkv, stage=64, direct=True)
    helpers.assert_parity(actual, expected, f"long interior runs hq={hq} hkv={hkv}")


@pytest.mark.parametrize("hq,hkv,d,tile,fp8", [(64, 8, 128, 32, False), (64, 8, 128, 16, False), (64, 8, 128, 32, True),
                                               (32, 4, 128, 16, True), (32, 8, 128, 4, False), (24, 4, 256, 16, False),
                                               (24, 4, 256, 16, True), (24, 4, 256, 32, False), (24, 4, 256, 32, True)])
def test_scores_that_keep_outgrowing_the_running_reference(device, hq, hkv, d, tile, fp8):
    """Every score of a sequence rises steadily along the context (by some 60 octaves over 3000 keys), so later scores
    exceed the earlier maximum by far more than any rescaling threshold, over and over: the reference-moving path of
    the tiles runs many times, in the masked head and tail tiles and in the interior ones, with direct output (whose
    two-column-tile builds at D 128 do not follow the largest score) and with partial states + Reduce (which must
    report it), on bf16 and FP8 pages."""
    histories = [0, 700, 2500]
    q_lens = [96, 64, 40]
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories,
                              q_lens=q_lens, seed=300 + tile, key_drift=0.04, fp8_pages=fp8)
    expected = helpers.expected_output(w)
    ratio = hq // hkv
    for kv_slice, direct in [(1 << 20, True), (1024, False)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, tile, kv_slice)
        print(f"growing scores hq={hq} hkv={hkv} d={d} tile={tile} fp8={fp8} kv_slice={kv_slice} direct={direct}", flush=True)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=tile,
                                         max_q_heads=ratio, stage=64, direct=direct)
        # On FP8 pages the drifting key dimension climbs in steps of an eighth of its value, so the weights pile up on the
        # few keys behind the latest step; single-rounded bf16 weights then show at 2-5e-3 on outputs of order one.  Still
        # four times tighter than the reference's own component tests (2e-2 per element, sliced_kv_test.rs:183,511-530).
        helpers.assert_parity(actual, expected, f"growing scores tile={tile} slice={kv_slice} direct={direct}",
                              abs_tol=5.0e-3 if fp8 else helpers.ABS_TOL)
