"""khm_sliced_kv_map_reduce_static: the fused decode Map + Reduce whose partial states and arrival counters live in the
library's static device array.  Through the C ABI, against khm_sliced_kv_map_reduce with caller buffers, bit for bit, on
two calls in a row (the second with a smaller input, so stale contents of the shared array would show), with and without
the gate; shapes beyond the array are rejected."""
import numpy as np
import pytest
import torch

from khalamari_amd import _lib, sdpa, sliced_kv
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, KhmError, ReplayU32
from oracle import gqa_oracle as oracle

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu


def _both(w, templates, cu, device, *, partial_dtype, gates=None):
    """(static-scratch output, caller-buffer output) as uint16 bit patterns."""
    g = w.geom
    config = gpu_runner.component_config(w, sliced_kv.Config, partial_dtype)
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), g.head_dim, 128, min(g.num_q_heads // g.num_kv_heads, 8))
    templates = np.asarray(templates, dtype=np.uint32).reshape(-1, 3)
    shape = sliced_kv.Shape(w.num_tokens, templates.shape[0])
    compute = sliced_kv.Compute(config, variant, shape)
    common = dict(q=gpu_runner.to_device(w.q_bits, device), kv_pages=gpu_runner.to_device(w.kv_pages, device),
                  req_slots=gpu_runner.to_device(w.req_slots, device), page_ids=gpu_runner.to_device(w.page_ids, device),
                  sdpa_map_task_templates=gpu_runner.to_device(templates, device),
                  cu_sdpa_partial_outputs=gpu_runner.to_device(np.asarray(cu, dtype=np.uint32), device),
                  page_table_index=ReplayU32.fixed(w.layer), num_active_tokens=ReplayU32.fixed(w.num_tokens),
                  num_active_kv_splits=ReplayU32.fixed(templates.shape[0]),
                  gates=gpu_runner.to_device(gates, device) if gates is not None else None)
    out_static = torch.full((w.num_tokens, g.num_q_heads, g.head_dim), 0x4228, dtype=torch.int16, device=device)
    compute.invoke_map_reduce_static(output=out_static, **common)
    scratch = sliced_kv.Scratch(device, config, shape)
    counters = torch.zeros(compute.arrival_counters_bytes(), dtype=torch.uint8, device=device)
    out_buffers = torch.full_like(out_static, 0x4228)
    compute.invoke_map_reduce(output=out_buffers, partial_exp_sums=scratch.partial_exp_sums,
                              partial_max_logits=scratch.partial_max_logits, partial_output=scratch.partial_output,
                              arrival_counters=counters, **common)
    torch.cuda.synchronize()
    return out_static.cpu().numpy().view(np.uint16), out_buffers.cpu().numpy().view(np.uint16)


def test_static_scratch_call_equals_the_call_with_caller_buffers(device):
    assert int(_lib.lib().khm_sliced_kv_static_scratch_bytes()) == 16 << 20
    cases = [
        # (histories, kv_slice, partial dtype, gated): a larger call first, a smaller one after it
        ([3000, 700, 4500, 33, 1500, 2047], 256, DTYPE_F32, False),
        ([900, 40], 512, DTYPE_F32, False),
        ([5000, 1200, 64], 256, DTYPE_BF16, True),
        ([300], 128, DTYPE_BF16, True),
    ]
    for number, (histories, kv_slice, partial_dtype, gated) in enumerate(cases):
        q_lens = [1] * len(histories)
        w = helpers.make_workload(num_q_heads=32, num_kv_heads=8, head_dim=128, tokens_per_page=16, histories=histories, q_lens=q_lens,
                                  seed=900 + number)
        _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, kv_slice)
        gates = None
        if gated:
            gates = oracle.f32_to_bf16_bits(np.random.default_rng(number).standard_normal((len(histories), 32, 128), dtype=np.float32))
        print(f"static scratch case {number}: histories={histories} slice={kv_slice} partial_dtype={partial_dtype} gated={gated}", flush=True)
        got, want = _both(w, templates, cu, device, partial_dtype=partial_dtype, gates=gates)
        assert np.array_equal(got, want), f"case {number}: {np.count_nonzero(got != want)} of {got.size} output values differ"
        expected = helpers.expected_output(w)
        if gated:
            expected = oracle.gate_f32(expected, oracle.bf16_bits_to_f32(gates))
        helpers.assert_parity(oracle.bf16_bits_to_f32(got), expected, f"static scratch case {number}", abs_tol=4e-3 if gated else helpers.ABS_TOL)


def test_static_scratch_rejects_shapes_beyond_the_array(device):
    layout = sliced_kv.Layout(1, 1, 8192, 1)
    config = sliced_kv.Config(64, 8, 128, 128 ** -0.5, 2 * 8 * 16 * 128 * 2, layout, DTYPE_BF16, DTYPE_BF16, DTYPE_F32)
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), 128, 128, 8)
    compute = sliced_kv.Compute(config, variant, sliced_kv.Shape(64, 1024))   # 1024 x 64 x 128 f32 = 32 MiB of partial outputs
    dummy = torch.zeros(64 * 64 * 128, dtype=torch.int16, device=device)
    small = torch.zeros(1024 * 3, dtype=torch.int32, device=device)
    pages = torch.zeros(config.page_bytes, dtype=torch.uint8, device=device)
    table = torch.zeros(8192, dtype=torch.int32, device=device)
    with pytest.raises(KhmError, match="static scratch"):
        compute.invoke_map_reduce_static(q=dummy, kv_pages=pages, req_slots=small, page_ids=table, sdpa_map_task_templates=small,
                                         cu_sdpa_partial_outputs=small, output=dummy, page_table_index=ReplayU32.fixed(0),
                                         num_active_tokens=ReplayU32.fixed(64), num_active_kv_splits=ReplayU32.fixed(1024))
    torch.cuda.synchronize()


def test_static_scratch_call_under_graph_capture_allocates_nothing(device):
    """The claims the entry point exists for: it can be recorded into a HIP graph (stream capture forbids allocation, so a
    hidden hipMalloc would fail the capture), device memory in use does not change across the call, and every replay -
    with eager work and synchronizations in between - equals the eager result."""
    histories = [1200, 300, 2047, 64]
    q_lens = [1] * len(histories)
    w = helpers.make_workload(num_q_heads=32, num_kv_heads=8, head_dim=128, tokens_per_page=16, histories=histories, q_lens=q_lens, seed=940)
    _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, 256)
    templates = np.asarray(templates, dtype=np.uint32).reshape(-1, 3)
    g = w.geom
    config = gpu_runner.component_config(w, sliced_kv.Config, DTYPE_BF16)
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), g.head_dim, 128, 4)
    compute = sliced_kv.Compute(config, variant, sliced_kv.Shape(w.num_tokens, templates.shape[0]))
    common = dict(q=gpu_runner.to_device(w.q_bits, device), kv_pages=gpu_runner.to_device(w.kv_pages, device),
                  req_slots=gpu_runner.to_device(w.req_slots, device), page_ids=gpu_runner.to_device(w.page_ids, device),
                  sdpa_map_task_templates=gpu_runner.to_device(templates, device),
                  cu_sdpa_partial_outputs=gpu_runner.to_device(np.asarray(cu, dtype=np.uint32), device),
                  page_table_index=ReplayU32.fixed(w.layer), num_active_tokens=ReplayU32.fixed(w.num_tokens),
                  num_active_kv_splits=ReplayU32.fixed(templates.shape[0]))
    out = torch.full((w.num_tokens, g.num_q_heads, g.head_dim), 0x4228, dtype=torch.int16, device=device)
    compute.invoke_map_reduce_static(output=out, **common)      # eager: the reference result, and the warm-up before capture
    torch.cuda.synchronize()
    eager = out.cpu().numpy().copy()
    helpers.assert_parity(oracle.bf16_bits_to_f32(eager.view(np.uint16)), helpers.expected_output(w), "static scratch, eager")

    free_before, _ = torch.cuda.mem_get_info(device)
    allocated_before = torch.cuda.memory_allocated(device)
    compute.invoke_map_reduce_static(output=out, **common)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(device)
    assert free_after == free_before and torch.cuda.memory_allocated(device) == allocated_before

    graph = gpu_runner.capture_graph(lambda: compute.invoke_map_reduce_static(output=out, **common))
    for replay in range(3):
        print(f"static scratch graph replay {replay}", flush=True)
        out.fill_(0x4228)           # eager fill kernel between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), eager), f"replay {replay} differs from the eager call"
