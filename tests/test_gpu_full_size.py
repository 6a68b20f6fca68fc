"""Parity at the full sizes of the five benchmark configs.  The synthetic configs are built exactly as bench.py builds them (same seeds,
page permutations and selector decisions), one step runs through the C ABI, and the output rows of sampled Q tokens are
checked against the CPU oracle at the full context - every token of configs 1 to 4, and 64 tokens of each request of
config 5, chosen so that every offset 0..31 inside a 32-token Q tile and 64 different tiles per request are hit (the
reference's bench gate samples first / middle / last: benches/gqa/matrix.rs:116-151).  Two size-independent properties close the gap for the rows the oracle does not visit:
the result does not depend on how the KV range is partitioned, and rows of unsampled tokens are finite and non-trivial."""
import numpy as np
import pytest
import torch

import bench
from oracle import gqa_oracle as oracle

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu


def _oracle_rows(workload, pool, tokens):
    """Oracle output rows [len(tokens), Hq, D] for flat Q token indices `tokens` of a bench workload."""
    spec = workload.spec
    hq, hkv, d = spec["hq"], spec["hkv"], spec["d"]
    table = workload.table_host
    geom = oracle.Geometry(hq, hkv, d, bench.TOKENS_PER_PAGE, d ** -0.5, 1, table.shape[1], 1,
                           oracle.KV_FP8_E4M3FN if workload.fp8_pages else oracle.KV_BF16)
    starts = np.concatenate([[0], np.cumsum(workload.q_lens)])
    slots, visible = [], []
    for token in tokens:
        request = int(np.searchsorted(starts, token, side="right") - 1)
        slots.append(request)
        visible.append((0, workload.histories[request] + (token - starts[request]) + 1))
    q_bits = workload.q[list(tokens)].cpu().view(torch.int16).numpy().view(np.uint16)
    pages = pool.cpu().view(torch.uint8).numpy() if pool.dtype == torch.uint8 else pool.cpu().view(torch.int16).numpy().view(np.uint8)
    return oracle.paged_gqa(geom, q_bits, pages, np.asarray(slots, dtype=np.uint32), table.reshape(-1),
                            np.asarray(visible, dtype=np.uint32), num_threads=16)


def _sampled_tokens(workload, per_request):
    """Flat Q token indices: every token of a request with at most `per_request` tokens (or per_request == 0), otherwise
    `per_request` of them: sample i sits at offset i % 32 of Q tile (i * 31) % tiles, plus the request's first and last."""
    starts = np.concatenate([[0], np.cumsum(workload.q_lens)])
    tokens = []
    for request, count in enumerate(workload.q_lens):
        if per_request == 0 or count <= per_request:
            picks = range(count)
        else:
            tiles = count // 32
            picks = sorted({0, count - 1} | {((i * 31) % tiles) * 32 + i % 32 for i in range(per_request)})
        tokens.extend(int(starts[request] + i) for i in picks)
    return tokens


def _run_step(workload, pool_index=0):
    workload.out.zero_()
    workload.launch_map(workload.kv_pools[pool_index])
    if workload.launch_reduce is not None:
        workload.launch_reduce()
    torch.cuda.synchronize()
    return gpu_runner.bf16_tensor_to_f32(workload.out.view(torch.int16))


@pytest.mark.parametrize("index,fp8", [(1, False), (2, False), (2, True), (3, False), (3, True)])
def test_decode_configs_at_full_size(device, index, fp8):
    workload = bench.Workload(index, device, num_pools=1, fp8_pages=fp8)
    actual = _run_step(workload)
    tokens = _sampled_tokens(workload, per_request=0)
    print(f"config {index} fp8={fp8}: oracle over {len(tokens)} tokens, {workload.visible_tokens} visible KV tokens", flush=True)
    expected = _oracle_rows(workload, workload.kv_pools[0], tokens)
    if workload.gates is not None:
        # config 3: the gate sees the bf16-rounded attention output (gqa_activation_gate.metal:19-39)
        gate_bits = workload.gates.cpu().view(torch.int16).numpy().view(np.uint16)[tokens]
        expected = oracle.bf16_bits_to_f32(oracle.gate_bf16(oracle.f32_to_bf16_bits(expected), gate_bits))
    stats = helpers.assert_parity(actual[tokens], expected, f"config {index} full size")
    print(stats)
    helpers.record_parity(f"config{index}{'_fp8_pages' if fp8 else ''} full size, bf16 output, {len(tokens)} tokens", stats)


@pytest.mark.parametrize("index,fp8", [(4, False), (4, True), (5, False), (5, True), (bench.EXTRA_PREFILL_D256, False),
                                       (bench.EXTRA_PREFILL_D256, True)])
def test_verify_and_prefill_configs_at_full_size(device, index, fp8):
    workload = bench.Workload(index, device, num_pools=1, fp8_pages=fp8)
    actual = _run_step(workload)
    assert np.isfinite(actual).all()
    assert (np.abs(actual).reshape(actual.shape[0], -1).max(axis=1) > 0).all()      # every token row was written
    tokens = _sampled_tokens(workload, per_request=64)
    print(f"config {index} fp8={fp8}: oracle over {len(tokens)} sampled tokens", flush=True)
    expected = _oracle_rows(workload, workload.kv_pools[0], tokens)
    stats = helpers.assert_parity(actual[tokens], expected, f"config {index} full size")
    print(stats)
    helpers.record_parity(f"{bench.config_key(index)}{'_fp8_pages' if fp8 else ''} full size, bf16 output, {len(tokens)} tokens", stats)


def test_partitioning_does_not_change_the_result_at_full_size(device):
    """Config 2 at full size with 512-token partitions, 2048-token partitions and unsplit: the same output up to the
    rounding of the bf16 partial states (the invariant of sdpa_test.rs:462-498 and docs/gqa_sdpa_selection.md:449-458)."""
    results = []
    for kv_slice in (512, 2048, 1 << 20):
        original = bench.CONFIGS[2]["kv_slice"]
        bench.CONFIGS[2]["kv_slice"] = kv_slice
        try:
            workload = bench.Workload(2, device, num_pools=1)
        finally:
            bench.CONFIGS[2]["kv_slice"] = original
        results.append(_run_step(workload))
        del workload
        torch.cuda.empty_cache()
    for other in results[1:]:
        helpers.assert_parity(other, results[0], "partition invariance")


@pytest.mark.parametrize("index", [1, 2, 4, 5])
def test_workload_is_released_without_the_cycle_collector(device, index):
    """A workload dropped by its owner gives back its pools and its metadata buffers (hipFree, hipHostFree) at once, by
    reference count.  Left to the cycle collector it would hold tens of gigabytes until some later allocation count is
    reached, and its frees could land inside another test's graph capture, which they would invalidate."""
    import gc
    import weakref

    gc.collect()
    gc.disable()
    try:
        workload = bench.Workload(index, device, num_pools=1)
        _run_step(workload)
        alive = [weakref.ref(workload), weakref.ref(workload.metadata), weakref.ref(workload.launch_map)]
        del workload
        assert [ref() for ref in alive] == [None, None, None]
    finally:
        gc.enable()
