"""A recorded launch sequence as a replay program: Map + Reduce captured once into a HIP graph whose kernels read
their active counts from a device parameter block, replayed with different arguments.  This is the HIP counterpart
of the reference's ReplayProgram + ReplayArguments (crates/inference-backend-metal/src/metal/stream/replay.rs:46-82,
submission.rs:124-135).  Every replay is checked against the eager launches and the oracle, with eager work and
synchronizations between the replays."""
import numpy as np
import pytest
import torch

from khalamari_amd import sdpa, sliced_kv, sliced_q
from khalamari_amd._lib import ReplayU32

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu

POISON = 0x4228


def test_decode_program_replays_with_different_active_counts(device):
    hq, hkv, d, tpp = 16, 2, 128, 16
    histories = [300, 17, 1000, 64, 0, 511, 77, 129]
    q_lens = [1] * len(histories)
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories, q_lens=q_lens, seed=61)
    _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, 128)
    tokens, total = len(histories), templates.shape[0]
    expected = helpers.expected_output(w)
    config = gpu_runner.component_config(w, sliced_kv.Config)
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), d, 128, 8)
    shape = sliced_kv.Shape(tokens, total)
    compute = sliced_kv.Compute(config, variant, shape)
    scratch = sliced_kv.Scratch(device, config, shape)
    dev = lambda a: gpu_runner.to_device(a, device)  # noqa: E731
    q, pages, slots, table, tmpl, cu_d = map(dev, (w.q_bits, w.kv_pages, w.req_slots, w.page_ids, templates, cu))
    params = torch.zeros(4, dtype=torch.int32, device=device)
    out = torch.full((tokens, hq, d), POISON, dtype=torch.int16, device=device)

    def record():
        compute.invoke_map(q=q, kv_pages=pages, req_slots=slots, page_ids=table, sdpa_map_task_templates=tmpl,
                           partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                           partial_output=scratch.partial_output, page_table_index=ReplayU32.fixed(0),
                           num_active_tokens=ReplayU32.parameter(0), num_active_kv_splits=ReplayU32.parameter(1), replay_parameters=params)
        compute.invoke_reduce(partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                              partial_output=scratch.partial_output, cu_sdpa_partial_outputs=cu_d, output=out,
                              num_active_tokens=ReplayU32.parameter(0), replay_parameters=params)

    def arguments(active_tokens):
        return torch.tensor([active_tokens, int(cu[active_tokens]), 0, 0], dtype=torch.int32)

    params.copy_(arguments(tokens))
    record()                       # eager warm-up before capture
    graph = gpu_runner.capture_graph(record)
    for active in [tokens, 1, 5, 3, 8, 2]:
        print(f"graph replay active={active}", flush=True)
        out.fill_(POISON)          # a fill kernel, eager, between replays
        params.copy_(arguments(active))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.fill_(POISON)
        record()                   # the same launches, eager
        torch.cuda.synchronize()
        assert torch.equal(replayed, out), f"replay differs from eager launches at active={active}"
        actual = gpu_runner.bf16_tensor_to_f32(replayed)
        helpers.assert_parity(actual[:active], expected[:active], f"graph replay active={active}")
        assert np.all(replayed[active:].cpu().numpy() == POISON)


def test_verify_program_replays_on_the_tiled_kernel(device):
    """The LDS-tiled kernel (dynamic LDS, direct-to-LDS loads) under graph capture: speculative-verify blocks."""
    hq, hkv, d = 32, 4, 128
    histories, q_lens = [300, 2000, 64, 900], [3, 5, 2, 4]
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories, q_lens=q_lens, seed=62)
    ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 8, 512)
    expected = helpers.expected_output(w)
    config = gpu_runner.component_config(w, sliced_q.Config)
    variant = sdpa.ExecutionVariant.sliced_q(config.sdpa_config(), sdpa.MAP_Q_TOKENS_AND_HEADS, 8, 64, 8)
    shape = sliced_q.Shape(w.num_tokens, ranges.shape[0], templates.shape[0])
    compute = sliced_q.Compute.new(config, variant, shape)
    dev = lambda a: gpu_runner.to_device(a, device)  # noqa: E731
    q, pages, slots, table, vis, rng_d, tmpl, cu_d = map(dev, (w.q_bits, w.kv_pages, w.req_slots, w.page_ids, w.visible, ranges, templates, cu))
    partial = torch.zeros(config.partial_output_bytes(variant, shape), dtype=torch.uint8, device=device)
    sums = torch.zeros(config.partial_output_stats_bytes(variant, shape), dtype=torch.uint8, device=device)
    maxs = torch.zeros_like(sums)
    params = torch.zeros(4, dtype=torch.int32, device=device)
    out = torch.full((w.num_tokens, hq, d), POISON, dtype=torch.int16, device=device)

    def record():
        compute.invoke_map(q=q, kv_pages=pages, req_slots=slots, page_ids=table, visible_kv_token_ranges=vis, q_token_ranges=rng_d,
                           sdpa_map_task_templates=tmpl, partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                           page_table_index=ReplayU32.fixed(0), num_active_tokens=ReplayU32.parameter(0),
                           num_active_q_token_tiles=ReplayU32.parameter(1), num_active_kv_splits=ReplayU32.parameter(2),
                           replay_parameters=params)
        compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=rng_d,
                              cu_sdpa_partial_outputs=cu_d, output=out, num_active_q_token_tiles=ReplayU32.parameter(1),
                              replay_parameters=params)

    def arguments(active_requests):
        active_tokens = int(sum(q_lens[:active_requests]))
        return active_tokens, torch.tensor([active_tokens, active_requests, int(cu[active_requests]), 0], dtype=torch.int32)

    params.copy_(arguments(len(q_lens))[1])
    record()
    graph = gpu_runner.capture_graph(record)
    for active_requests in [4, 1, 3, 2, 4]:
        active_tokens, block = arguments(active_requests)
        print(f"verify graph replay requests={active_requests}", flush=True)
        out.fill_(POISON)
        params.copy_(block)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.fill_(POISON)
        record()
        torch.cuda.synchronize()
        assert torch.equal(replayed, out)
        actual = gpu_runner.bf16_tensor_to_f32(replayed)
        helpers.assert_parity(actual[:active_tokens], expected[:active_tokens], f"verify graph replay requests={active_requests}")
        assert np.all(replayed[active_tokens:].cpu().numpy() == POISON)
